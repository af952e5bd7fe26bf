// linear_wide.h's kernels for the gated epilogue and up to 128 rows.
#include "linear_wide.h"

PALM_WIDE_INSTANCE(wide_launch_gated_128, 8, WIDE_SWIGLU)
