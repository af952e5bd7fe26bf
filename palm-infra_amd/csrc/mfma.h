// Matrix-core (MFMA) building blocks for gfx950, bfloat16 inputs and 32-bit accumulation.
//
// v_mfma_f32_16x16x32_bf16: D[16x16] += A[16x32] . B[32x16].  Register layout, lane l = 16 g + r:
//   A: lane holds row r,    eight k-values of group g        (8 bf16 = 16 bytes)
//   B: lane holds column r, the same eight k-values of group g
//   D: lane holds column r, rows 4 g .. 4 g + 3               (4 floats)
// A dot product does not care in which order k is visited, so as long as A and B give a lane the same
// k-values, any assignment of k to (group, element) is right.  The kernels use that to let each lane
// read long contiguous runs of a row.
#pragma once

#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ inline f32x4 mfma_16x16x32(bf16x8 a, bf16x8 b, f32x4 acc) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
}

__device__ inline bf16x8 load_bf16x8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }

__device__ inline bf16x8 zero_bf16x8() {
    bf16x8 z;
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
    return z;
}
