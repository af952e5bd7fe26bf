// C[M, N] = A[M, K] . W[N, K]^T for few rows (decode steps, logits rows): bfloat16 operands on the matrix
// cores, 32-bit accumulation, the weight streamed from HBM once per 64 rows of A.  The product itself is the
// reference's matmul (kernels/matmul_dense.cpp:939-953); its GEMV paths (kernels/matmul_dense.cpp:1282-1332)
// are what this kernel stands for.  An epilogue can apply the gated activation of the feed-forward
// (out = silu(gate) * up, engine/cuda_ops.cu:100-112) so that the [M, 2I] product never goes to memory.
//
// Work split.  A block owns RT strips of 16 weight rows (16 output features each) and all of K; its waves
// take every NW-th "super-step" of 128 k-values and their partial tiles are added in LDS in a fixed order (no
// atomics: the same input gives the same bits).  In a super-step lane (r, g) of a wave makes four 16-byte
// reads of weight row r of each strip, at k = k0 + 32 j + 8 g for j = 0..3, so that each read instruction
// takes 64 contiguous bytes of every row (the four lanes of a row side by side) and the four together a run
// of 256 bytes; it reads the same k-values of activation row r for each block of 16 tokens, once for all RT
// strips, and MFMA 16x16x32 consume them.  Several super-steps are loaded before any is used, which is what
// keeps enough bytes in flight to fill the memory pipe with only one or two blocks on a compute unit.
// RT = 2 halves the activation reads per weight byte but was measured slower; RT = 1 is what runs.
#include "mfma.h"

enum ThinEpilogue : int { EPI_STORE = 0, EPI_SWIGLU = 1 };

constexpr int SUPER_K = 128;

template <int MB, int NW, int U, int RT, typename TC, int EPI>
__global__ __launch_bounds__(NW * WAVE) void linear_thin_kernel(const bf16_t* __restrict__ A,
                                                                const bf16_t* __restrict__ W, TC* __restrict__ C,
                                                                int M, int N, int K) {
    __shared__ float part[NW][RT][MB][16][17];
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    const int r = lane % 16, g = lane / 16;
    const int tok0 = blockIdx.y * MB * 16;
    const int inter = N / 2;

    // the weight rows this lane reads: one in each of the block's strips
    const bf16_t* wp[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int strip = blockIdx.x * RT + rt;
        int wrow;
        if (EPI == EPI_SWIGLU) wrow = (r < 8 ? 0 : inter) + min(strip * 8 + (r % 8), inter - 1);   // 8 gate rows, their 8 up rows
        else wrow = min(strip * 16 + r, N - 1);
        wp[rt] = W + (size_t)wrow * K + g * 8;
    }
    const bf16_t* xp[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) xp[mb] = A + (size_t)min(tok0 + mb * 16 + r, M - 1) * K + g * 8;

    f32x4 acc[RT][MB];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[rt][mb] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int n_super = (K + SUPER_K - 1) / SUPER_K;
    for (int ss = wave; ss < n_super; ss += NW * U) {
        bf16x8 wv[U][RT][4];
        bf16x8 xv[U][MB][4];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k0 = (ss + u * NW) * SUPER_K;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bool ok = k0 + j * 32 + g * 8 < K;            // K is a multiple of 8: a chunk is whole or absent
                const int at = ok ? k0 + j * 32 : 0;                // an absent chunk reads the row's start and is zeroed
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    const bf16x8 v = load_bf16x8(wp[rt] + at);
                    wv[u][rt][j] = ok ? v : zero_bf16x8();
                }
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const bf16x8 v = load_bf16x8(xp[mb] + at);
                    xv[u][mb][j] = ok ? v : zero_bf16x8();
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) acc[rt][mb] = mfma_16x16x32(wv[u][rt][j], xv[u][mb][j], acc[rt][mb]);
    }

    // D: this lane holds token column r, weight rows 4 g + i
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 4; ++i) part[wave][rt][mb][4 * g + i][r] = acc[rt][mb][i];
    __syncthreads();

    if (EPI == EPI_SWIGLU) {
        for (int idx = threadIdx.x; idx < RT * MB * 128; idx += NW * WAVE) {
            const int rt = idx / (MB * 128), mb = (idx / 128) % MB, c = idx % 8, col = (idx % 128) / 8;
            float gate = 0.f, up = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) { gate += part[w][rt][mb][c][col]; up += part[w][rt][mb][c + 8][col]; }
            const int tok = tok0 + mb * 16 + col, feat = (blockIdx.x * RT + rt) * 8 + c;
            if (tok < M && feat < inter) C[(size_t)tok * inter + feat] = from_float<TC>(gate / (1.0f + expf(-gate)) * up);
        }
    } else {
        for (int idx = threadIdx.x; idx < RT * MB * 256; idx += NW * WAVE) {
            const int rt = idx / (MB * 256), mb = (idx / 256) % MB, row = idx % 16, col = (idx % 256) / 16;
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) v += part[w][rt][mb][row][col];
            const int tok = tok0 + mb * 16 + col, feat = (blockIdx.x * RT + rt) * 16 + row;
            if (tok < M && feat < N) C[(size_t)tok * N + feat] = from_float<TC>(v);
        }
    }
}

template <int MB, int NW, int U, int RT, typename TC, int EPI>
static void launch_thin(hipStream_t stream, const void* a, const void* w, void* c, int M, int N, int K) {
    const int strips = EPI == EPI_SWIGLU ? (N / 2 + 7) / 8 : (N + 15) / 16;
    dim3 grid((strips + RT - 1) / RT, (M + MB * 16 - 1) / (MB * 16));
    linear_thin_kernel<MB, NW, U, RT, TC, EPI><<<grid, NW * WAVE, 0, stream>>>(
        (const bf16_t*)a, (const bf16_t*)w, (TC*)c, M, N, K);
}

template <typename TC, int EPI>
static void dispatch_thin(hipStream_t stream, const void* a, const void* w, void* c, int M, int N, int K) {
    const bool deep = (K + SUPER_K - 1) / SUPER_K >= 16;       // enough super-steps to feed eight waves
    if (M <= 16) {
        // eight waves, two super-steps in flight each, two blocks on a compute unit: measured best
        // (two strips a block, RT = 2, were measured slower at every size: 50.6 against 43.1 us for the gated
        // product at 8 rows, 327 against 243 us for the head)
        if (deep) launch_thin<1, 8, 2, 1, TC, EPI>(stream, a, w, c, M, N, K);
        else launch_thin<1, 4, 2, 1, TC, EPI>(stream, a, w, c, M, N, K);
    } else if (M <= 32) {
        if (deep) launch_thin<2, 8, 2, 1, TC, EPI>(stream, a, w, c, M, N, K);
        else launch_thin<2, 4, 2, 1, TC, EPI>(stream, a, w, c, M, N, K);
    } else {
        if (deep) launch_thin<4, 8, 2, 1, TC, EPI>(stream, a, w, c, M, N, K);
        else launch_thin<4, 4, 1, 1, TC, EPI>(stream, a, w, c, M, N, K);
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
