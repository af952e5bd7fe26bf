// linear_wide.h's kernels for the gated epilogue and up to 64 rows.
#include "linear_wide.h"

PALM_WIDE_INSTANCE(wide_launch_gated_64, 4, WIDE_SWIGLU)
