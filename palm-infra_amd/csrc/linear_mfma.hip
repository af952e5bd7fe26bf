// C[M, N] = A[M, K] . W[N, K]^T for few rows (decode steps, logits rows): bfloat16 operands on the matrix
// cores, 32-bit accumulation, the weight streamed from HBM once per 64 rows of A.  The product itself is the
// reference's matmul (kernels/matmul_dense.cpp:939-953); its GEMV paths (kernels/matmul_dense.cpp:1282-1332)
// are what this kernel stands for.  An epilogue can apply the gated activation of the feed-forward
// (out = silu(gate) * up, engine/cuda_ops.cu:100-112) so that the [M, 2I] product never goes to memory.
//
// Work split.  A block owns a strip of 16 weight rows (16 output features) and all of K; its waves take
// every NW-th "super-step" of 128 k-values and their partial tiles are added in LDS in a fixed order (no
// atomics: the same input gives the same bits).  In a super-step lane (r, g) of a wave makes four 16-byte
// reads of weight row r, at k = k0 + 32 j + 8 g for j = 0..3, so that each read instruction takes 64
// contiguous bytes of every row (the four lanes of a row side by side) and the four together a run of 256
// bytes; it reads the same k-values of activation row r for each block of 16 tokens, and four MFMA 16x16x32
// consume them.  Several super-steps are loaded before any is used, which is what keeps enough bytes in
// flight to fill the memory pipe with only one or two blocks on a compute unit.
#include "mfma.h"

enum ThinEpilogue : int { EPI_STORE = 0, EPI_SWIGLU = 1 };

constexpr int SUPER_K = 128;

template <int MB, int NW, int U, typename TC, int EPI>
__global__ __launch_bounds__(NW * WAVE) void linear_thin_kernel(const bf16_t* __restrict__ A,
                                                                const bf16_t* __restrict__ W, TC* __restrict__ C,
                                                                int M, int N, int K) {
    __shared__ float part[NW][MB][16][17];
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    const int r = lane % 16, g = lane / 16;
    const int strip = blockIdx.x;
    const int tok0 = blockIdx.y * MB * 16;

    // the weight row this lane reads
    int wrow;
    if (EPI == EPI_SWIGLU) {
        const int inter = N / 2;                         // W is [gate rows | up rows]; the strip is 8 of each
        const int c = strip * 8 + (r % 8);
        wrow = (r < 8 ? 0 : inter) + min(c, inter - 1);
    } else {
        wrow = min(strip * 16 + r, N - 1);
    }
    const bf16_t* wp = W + (size_t)wrow * K + g * 8;
    const bf16_t* xp[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) xp[mb] = A + (size_t)min(tok0 + mb * 16 + r, M - 1) * K + g * 8;

    f32x4 acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int n_super = (K + SUPER_K - 1) / SUPER_K;
    for (int ss = wave; ss < n_super; ss += NW * U) {
        bf16x8 wv[U][4];
        bf16x8 xv[U][MB][4];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k0 = (ss + u * NW) * SUPER_K;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bool ok = k0 + j * 32 + g * 8 < K;            // K is a multiple of 8: a chunk is whole or absent
                wv[u][j] = ok ? load_bf16x8(wp + k0 + j * 32) : zero_bf16x8();
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) xv[u][mb][j] = ok ? load_bf16x8(xp[mb] + k0 + j * 32) : zero_bf16x8();
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) acc[mb] = mfma_16x16x32(wv[u][j], xv[u][mb][j], acc[mb]);
    }

    // D: this lane holds token column r, weight rows 4 g + i
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int i = 0; i < 4; ++i) part[wave][mb][4 * g + i][r] = acc[mb][i];
    __syncthreads();

    if (EPI == EPI_SWIGLU) {
        const int inter = N / 2;
        for (int idx = threadIdx.x; idx < MB * 128; idx += NW * WAVE) {
            const int mb = idx / 128, c = idx % 8, col = (idx % 128) / 8;
            float gate = 0.f, up = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) { gate += part[w][mb][c][col]; up += part[w][mb][c + 8][col]; }
            const int tok = tok0 + mb * 16 + col, feat = strip * 8 + c;
            if (tok < M && feat < inter) C[(size_t)tok * inter + feat] = from_float<TC>(gate / (1.0f + expf(-gate)) * up);
        }
    } else {
        for (int idx = threadIdx.x; idx < MB * 256; idx += NW * WAVE) {
            const int mb = idx / 256, row = idx % 16, col = (idx % 256) / 16;
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) v += part[w][mb][row][col];
            const int tok = tok0 + mb * 16 + col, feat = strip * 16 + row;
            if (tok < M && feat < N) C[(size_t)tok * N + feat] = from_float<TC>(v);
        }
    }
}

template <int MB, int NW, int U, typename TC, int EPI>
static void launch_thin(hipStream_t stream, const void* a, const void* w, void* c, int M, int N, int K) {
    const int strips = EPI == EPI_SWIGLU ? (N / 2 + 7) / 8 : (N + 15) / 16;
    dim3 grid(strips, (M + MB * 16 - 1) / (MB * 16));
    linear_thin_kernel<MB, NW, U, TC, EPI><<<grid, NW * WAVE, 0, stream>>>(
        (const bf16_t*)a, (const bf16_t*)w, (TC*)c, M, N, K);
}

template <typename TC, int EPI>
static void dispatch_thin(hipStream_t stream, const void* a, const void* w, void* c, int M, int N, int K) {
    const bool deep = (K + SUPER_K - 1) / SUPER_K >= 16;       // enough super-steps to feed eight waves
    if (M <= 16) {
        if (deep) launch_thin<1, 8, 2, TC, EPI>(stream, a, w, c, M, N, K);      // two super-steps in flight a wave, two blocks a CU: measured best
        else launch_thin<1, 4, 2, TC, EPI>(stream, a, w, c, M, N, K);
    } else if (M <= 32) {
        if (deep) launch_thin<2, 8, 2, TC, EPI>(stream, a, w, c, M, N, K);
        else launch_thin<2, 4, 2, TC, EPI>(stream, a, w, c, M, N, K);
    } else {
        if (deep) launch_thin<4, 8, 2, TC, EPI>(stream, a, w, c, M, N, K);
        else launch_thin<4, 4, 1, TC, EPI>(stream, a, w, c, M, N, K);
    }
}

// a [M, K] bfloat16, w [N, K] bfloat16; c [M, N] (EPI_STORE) or [M, N/2] (EPI_SWIGLU) in bfloat16 or float32.
PALM_API int palm_linear_thin(hipStream_t stream, const void* a, const void* w, void* c, int c_dtype, int M, int N,
                              int K, int epilogue) {
    PALM_CHECK(M >= 0 && N > 0 && K > 0, "linear_thin: M=%d N=%d K=%d", M, N, K);
    PALM_CHECK(K % 8 == 0, "linear_thin: K = %d is not a multiple of 8 (rows must start on 16 bytes)", K);
    PALM_CHECK(epilogue == EPI_STORE || epilogue == EPI_SWIGLU, "linear_thin: epilogue %d", epilogue);
    PALM_CHECK(epilogue != EPI_SWIGLU || N % 2 == 0, "linear_thin: a gated product needs an even N, got %d", N);
    PALM_CHECK(((uintptr_t)a | (uintptr_t)w) % 16 == 0, "linear_thin: operands must be 16-byte aligned");
    if (M == 0) return 0;
    PALM_CHECK((M + 63) / 64 <= 65535, "linear_thin: M=%d is more than one launch takes", M);
    if (epilogue == EPI_SWIGLU) {
        PALM_DTYPE_SWITCH(c_dtype, TC, dispatch_thin<TC, EPI_SWIGLU>(stream, a, w, c, M, N, K));
    } else {
        PALM_DTYPE_SWITCH(c_dtype, TC, dispatch_thin<TC, EPI_STORE>(stream, a, w, c, M, N, K));
    }
    PALM_LAUNCHED();
    return 0;
}
