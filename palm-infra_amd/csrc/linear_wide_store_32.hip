// linear_wide.h's kernels for the plain epilogue and up to 32 rows.
#include "linear_wide.h"

PALM_WIDE_INSTANCE(wide_launch_store_32, 2, WIDE_STORE)
