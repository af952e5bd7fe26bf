// C[M, N] (+)= A[M, K] . W[N, K]^T with W in the checkpoint's [out, in] layout and 32-bit accumulation
// (kernels/matmul_dense.cpp:939-953 gives the semantics; the reference's GPU path calls a library
// with 32-bit compute, engine/cuda_matmul.cu:245-260).
//
// This is the exact path: plain FMA in 32-bit, no matrix-core mode of reduced precision.  Every output
// element adds its products in the same order of k whatever M and N are, so a row's result does not
// depend on how many rows are computed with it.  The sum goes in two levels, runs of SUM_RUN products and then
// the runs' sums: a 32-bit sum of K terms one after the other is off by about sqrt(K) roundings, which at
// K = 12288 and 36 layers adds up to more than 1e-4 on logits of order one; two levels leave
// sqrt(SUM_RUN) + sqrt(K / SUM_RUN).  It serves the float32 mode and any mix of element
// types (a 32-bit matrix under bfloat16 activations).
#include "common.h"

constexpr int TILE_M = 64, TILE_N = 64, TILE_K = 16;
constexpr int SUM_RUN = 256;          // products added one after the other before their sum joins the total
static_assert(SUM_RUN % TILE_K == 0, "a run is a whole number of tiles");

template <typename TA, typename TW, typename TC>
__global__ __launch_bounds__(256) void linear_tiled_kernel(const TA* __restrict__ A, const TW* __restrict__ W,
                                                          TC* __restrict__ C, int M, int N, int K, int accumulate) {
    // k-major tiles so that a thread's four rows (columns) are one 16-byte read
    __shared__ float As[TILE_K][TILE_M + 4];
    __shared__ float Ws[TILE_K][TILE_N + 4];
    const int tid = threadIdx.x;
    const int tx = tid % 16, ty = tid / 16;          // thread computes rows ty*4.., columns tx*4..
    const int m0 = blockIdx.y * TILE_M, n0 = blockIdx.x * TILE_N;
    const int lrow = tid / 4, lk = (tid % 4) * 4;    // what this thread loads: one row, four k
    float acc[4][4] = {}, total[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += TILE_K) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + lk + j;
            const int m = m0 + lrow, n = n0 + lrow;
            As[lk + j][lrow] = (m < M && k < K) ? to_float(A[(size_t)m * K + k]) : 0.f;
            Ws[lk + j][lrow] = (n < N && k < K) ? to_float(W[(size_t)n * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < TILE_K; ++k) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { a[i] = As[k][ty * 4 + i]; w[i] = Ws[k][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        if ((k0 + TILE_K) % SUM_RUN == 0 || k0 + TILE_K >= K) {      // the run is over: its sum joins the total
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) { total[i][j] += acc[i][j]; acc[i][j] = 0.f; }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = total[i][j];
            if (accumulate) v += to_float(C[(size_t)m * N + n]);
            C[(size_t)m * N + n] = from_float<TC>(v);
        }
    }
}

PALM_API int palm_linear(hipStream_t stream, const void* a, int a_dtype, const void* w, int w_dtype, void* c,
                         int c_dtype, int M, int N, int K, int accumulate) {
    PALM_CHECK(M >= 0 && N > 0 && K > 0, "linear: M=%d N=%d K=%d", M, N, K);
    if (M == 0) return 0;
    dim3 grid((N + TILE_N - 1) / TILE_N, (M + TILE_M - 1) / TILE_M);
    PALM_CHECK(grid.y <= 65535, "linear: M=%d is more than one launch takes (%d rows)", M, 65535 * TILE_M);
    PALM_DTYPE_SWITCH(a_dtype, TA, PALM_DTYPE_SWITCH(w_dtype, TW, PALM_DTYPE_SWITCH(c_dtype, TC,
        linear_tiled_kernel<TA, TW, TC><<<grid, 256, 0, stream>>>(
            (const TA*)a, (const TW*)w, (TC*)c, M, N, K, accumulate))));
    PALM_LAUNCHED();
    return 0;
}
