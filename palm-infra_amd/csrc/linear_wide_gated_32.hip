// linear_wide.h's kernels for the gated epilogue and up to 32 rows.
#include "linear_wide.h"

PALM_WIDE_INSTANCE(wide_launch_gated_32, 2, WIDE_SWIGLU)
