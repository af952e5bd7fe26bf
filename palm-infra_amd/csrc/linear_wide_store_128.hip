// linear_wide.h's kernels for the plain epilogue and up to 128 rows.
#include "linear_wide.h"

PALM_WIDE_INSTANCE(wide_launch_store_128, 8, WIDE_STORE)
