// C[M, N] = A[M, K] . W[N, K]^T for 17 to some hundred rows (decode steps of large batches): bfloat16 on the
// matrix cores, 32-bit accumulation.  The thin kernel (linear_mfma.hip) lets every wave fetch the activations
// it needs straight from the caches, which for more than 16 rows is several times the weight traffic; here a
// block of four waves shares them through LDS.
//
// A block owns 64 weight rows (one strip of 16 for each wave), a tile of MB*16 rows of A, and a range of K
// (grid.y splits K when there are too few row tiles to fill the chip; the partial results then go to a
// workspace and a second kernel adds them in a fixed order).  Per step of 128 k-values the block copies the
// activation tile into LDS once (double buffered: one barrier a step); each wave reads its weight fragments
// from memory, 64 contiguous bytes of a row per instruction as in the thin kernel, and its B operands from
// LDS.  The next step's reads are issued before the current step's products.
// With the gated epilogue (out = silu(gate) * up, engine/cuda_ops.cu:100-112) a wave's strip is eight gate
// rows and the eight up rows that belong to them.
#include "mfma.h"

enum WideEpilogue : int { WIDE_STORE = 0, WIDE_SWIGLU = 1 };

constexpr int WIDE_K = 128;                     // k-values a step
constexpr int X_STRIDE = WIDE_K + 8;            // padded rows: the eight lanes LDS serves together hit different banks
constexpr int WIDE_WAVES = 4;

template <int MB, typename TC, int EPI>
__global__ __launch_bounds__(WIDE_WAVES * WAVE) void linear_wide_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, TC* __restrict__ C, float* __restrict__ work,
    int M, int N, int K, int steps_per_split) {
    __shared__ __attribute__((aligned(16))) bf16_t x_lds[2][MB * 16 * X_STRIDE];
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, r = lane % 16, g = lane / 16;
    const int split = blockIdx.y, n_splits = gridDim.y;
    const int tok0 = blockIdx.z * MB * 16;
    const int inter = N / 2;

    // the weight row this lane reads, and the feature its results belong to
    const int strip = blockIdx.x * WIDE_WAVES + wave;
    int wrow;
    if (EPI == WIDE_SWIGLU) wrow = (r < 8 ? 0 : inter) + min(strip * 8 + (r % 8), inter - 1);
    else wrow = min(strip * 16 + r, N - 1);
    const bf16_t* wp = W + (size_t)wrow * K + g * 8;

    const int n_steps = (K + WIDE_K - 1) / WIDE_K;
    const int s0 = split * steps_per_split, s1 = min(n_steps, s0 + steps_per_split);

    f32x4 acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};

    // what a thread copies of the activation tile: MB chunks of 16 bytes (the tile has MB*16 rows of 16 chunks)
    bf16x8 xr[MB], wr[4];
    auto fetch = [&](int step) {
        const int k0 = step * WIDE_K;
#pragma unroll
        for (int i = 0; i < MB; ++i) {
            const int c = i * (WIDE_WAVES * WAVE) + threadIdx.x, row = c / 16, ch = c % 16;
            const bool ok = k0 + ch * 8 < K;
            const bf16x8 v = load_bf16x8(A + (size_t)min(tok0 + row, M - 1) * K + (ok ? k0 + ch * 8 : 0));
            xr[i] = ok ? v : zero_bf16x8();
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bool ok = k0 + j * 32 + g * 8 < K;
            const bf16x8 v = load_bf16x8(wp + (ok ? k0 + j * 32 : 0));
            wr[j] = ok ? v : zero_bf16x8();
        }
    };

    if (s0 < s1) fetch(s0);
    int buf = 0;
    for (int step = s0; step < s1; ++step) {
#pragma unroll
        for (int i = 0; i < MB; ++i) {
            const int c = i * (WIDE_WAVES * WAVE) + threadIdx.x;
            *reinterpret_cast<bf16x8*>(&x_lds[buf][(c / 16) * X_STRIDE + (c % 16) * 8]) = xr[i];
        }
        bf16x8 wc[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) wc[j] = wr[j];
        __syncthreads();                                   // the tile is whole; the other buffer is free again
        if (step + 1 < s1) fetch(step + 1);                // on its way while this step's products run
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                const bf16x8 xf = *reinterpret_cast<const bf16x8*>(&x_lds[buf][(mb * 16 + r) * X_STRIDE + (j * 4 + g) * 8]);
                acc[mb] = mfma_16x16x32(wc[j], xf, acc[mb]);
            }
        buf ^= 1;
    }

    // this lane holds token column r of each block mb, weight rows 4g + i of the wave's strip
    if (n_splits > 1) {
        // raw partial sums, [split][token][weight row]; the second kernel adds them and applies the epilogue
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            const int tok = tok0 + mb * 16 + r;
            if (tok >= M) continue;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = 4 * g + i;
                int feat;
                if (EPI == WIDE_SWIGLU) feat = (row < 8 ? 0 : inter) + strip * 8 + row % 8;
                else feat = strip * 16 + row;
                const bool ok = EPI == WIDE_SWIGLU ? strip * 8 + row % 8 < inter : feat < N;
                if (ok) work[((size_t)split * M + tok) * N + feat] = acc[mb][i];
            }
        }
        return;
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int tok = tok0 + mb * 16 + r;
        if (EPI == WIDE_SWIGLU) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float up = __shfl(acc[mb][i], (lane + 32) % WAVE, WAVE);     // row 4g+i+8 lives 32 lanes on
                const int feat = strip * 8 + 4 * g + i;
                if (g < 2 && tok < M && feat < inter) {
                    const float gate = acc[mb][i];
                    C[(size_t)tok * inter + feat] = from_float<TC>(gate / (1.0f + expf(-gate)) * up);
                }
            }
        } else {
            if (tok >= M) continue;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int feat = strip * 16 + 4 * g + i;
                if (feat < N) C[(size_t)tok * N + feat] = from_float<TC>(acc[mb][i]);
            }
        }
    }
}

// out[m][n] = sum over splits, in order; with the gated epilogue out[m][c] = silu(sum gate) * sum up
template <typename TC, int EPI>
__global__ void linear_wide_reduce_kernel(const float* __restrict__ work, TC* __restrict__ C, int M, int N, int n_splits) {
    const int out_cols = EPI == WIDE_SWIGLU ? N / 2 : N;
    const size_t total = (size_t)M * out_cols;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
        const size_t m = idx / out_cols, c = idx % out_cols;
        float a = 0.f, b = 0.f;
        for (int s = 0; s < n_splits; ++s) {
            const float* row = work + ((size_t)s * M + m) * N;
            a += row[c];
            if (EPI == WIDE_SWIGLU) b += row[N / 2 + c];
        }
        C[idx] = from_float<TC>(EPI == WIDE_SWIGLU ? a / (1.0f + expf(-a)) * b : a);
    }
}

// Into how many ranges K is split: one if the row tiles alone fill the chip, else enough for about 512 blocks,
// each with at least two steps.
PALM_API int palm_linear_wide_splits(int M, int N, int K, int epilogue) {
    const int mb = M <= 32 ? 2 : 4;
    const int row_tiles = epilogue == WIDE_SWIGLU ? (N / 2 + 31) / 32 : (N + 63) / 64;
    const int blocks = row_tiles * ((M + mb * 16 - 1) / (mb * 16));
    const int n_steps = (K + WIDE_K - 1) / WIDE_K;
    if (blocks >= 256) return 1;
    int splits = (512 + blocks - 1) / blocks;
    if (splits > n_steps / 2) splits = n_steps / 2;
    return splits < 1 ? 1 : splits;
}

template <int MB, typename TC, int EPI>
static void launch_wide(hipStream_t stream, const void* a, const void* w, void* c, float* work, int M, int N, int K,
                        int splits) {
    const int row_tiles = EPI == WIDE_SWIGLU ? (N / 2 + 31) / 32 : (N + 63) / 64;
    const int n_steps = (K + WIDE_K - 1) / WIDE_K;
    const int per = (n_steps + splits - 1) / splits;
    dim3 grid(row_tiles, splits, (M + MB * 16 - 1) / (MB * 16));
    linear_wide_kernel<MB, TC, EPI><<<grid, WIDE_WAVES * WAVE, 0, stream>>>(
        (const bf16_t*)a, (const bf16_t*)w, (TC*)c, work, M, N, K, per);
    if (splits > 1) {
        const size_t total = (size_t)M * (EPI == WIDE_SWIGLU ? N / 2 : N);
        const int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
        linear_wide_reduce_kernel<TC, EPI><<<blocks, 256, 0, stream>>>(work, (TC*)c, M, N, splits);
    }
}

// a [M, K] bfloat16, w [N, K] bfloat16; c [M, N] (store) or [M, N/2] (gated) in bfloat16 or float32;
// work: splits * M * N floats if splits > 1 (splits as palm_linear_wide_splits says, or fewer).
PALM_API int palm_linear_wide(hipStream_t stream, const void* a, const void* w, void* c, int c_dtype, int M, int N, int K,
                              int epilogue, int splits, float* work) {
    PALM_CHECK(M >= 0 && N > 0 && K > 0, "linear_wide: M=%d N=%d K=%d", M, N, K);
    PALM_CHECK(K % 8 == 0, "linear_wide: K = %d is not a multiple of 8 (rows must start on 16 bytes)", K);
    PALM_CHECK(epilogue == WIDE_STORE || epilogue == WIDE_SWIGLU, "linear_wide: epilogue %d", epilogue);
    PALM_CHECK(epilogue != WIDE_SWIGLU || N % 2 == 0, "linear_wide: a gated product needs an even N, got %d", N);
    PALM_CHECK(((uintptr_t)a | (uintptr_t)w) % 16 == 0, "linear_wide: operands must be 16-byte aligned");
    PALM_CHECK(splits >= 1 && splits <= 65535 && (splits == 1 || work), "linear_wide: %d splits need a workspace", splits);
    if (M == 0) return 0;
    PALM_CHECK((M + 31) / 32 <= 65535, "linear_wide: M=%d is more than one launch takes", M);
    if (M <= 32) {
        if (epilogue == WIDE_SWIGLU) { PALM_DTYPE_SWITCH(c_dtype, TC, launch_wide<2, TC, WIDE_SWIGLU>(stream, a, w, c, work, M, N, K, splits)); }
        else { PALM_DTYPE_SWITCH(c_dtype, TC, launch_wide<2, TC, WIDE_STORE>(stream, a, w, c, work, M, N, K, splits)); }
    } else {
        if (epilogue == WIDE_SWIGLU) { PALM_DTYPE_SWITCH(c_dtype, TC, launch_wide<4, TC, WIDE_SWIGLU>(stream, a, w, c, work, M, N, K, splits)); }
        else { PALM_DTYPE_SWITCH(c_dtype, TC, launch_wide<4, TC, WIDE_STORE>(stream, a, w, c, work, M, N, K, splits)); }
    }
    PALM_LAUNCHED();
    return 0;
}
