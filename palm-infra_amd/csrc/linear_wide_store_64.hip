// linear_wide.h's kernels for the plain epilogue and up to 64 rows.
#include "linear_wide.h"

PALM_WIDE_INSTANCE(wide_launch_store_64, 4, WIDE_STORE)
