// C[M, N] = A[M, K] . W[N, K]^T for up to 16 rows (decode steps, logits rows): bfloat16 operands on the matrix
// cores, 32-bit accumulation, the weight streamed from HBM once.  The product itself is the
// reference's matmul (kernels/matmul_dense.cpp:939-953); its GEMV paths (kernels/matmul_dense.cpp:1282-1332)
// are what this kernel stands for.  An epilogue can apply the gated activation of the feed-forward
// (out = silu(gate) * up, engine/cuda_ops.cu:100-112) so that the [M, 2I] product never goes to memory.
//
// Two kernels: for a short K the one described next, for a long K the stream kernel further down.
// Work split.  A block owns RT strips of 16 weight rows (16 output features each) and all of K; its waves
// take every NW-th "super-step" of 128 k-values and their partial tiles are added in LDS in a fixed order (no
// atomics: the same input gives the same bits).  In a super-step lane (r, g) of a wave makes four 16-byte
// reads of weight row r of each strip, at k = k0 + 32 j + 8 g for j = 0..3, so that each read instruction
// takes 64 contiguous bytes of every row (the four lanes of a row side by side) and the four together a run
// of 256 bytes; it reads the same k-values of activation row r for each block of 16 tokens, once for all RT
// strips, and MFMA 16x16x32 consume them.  Several super-steps are loaded before any is used, which is what
// keeps enough bytes in flight to fill the memory pipe with only one or two blocks on a compute unit.
// RT = 2 halves the activation reads per weight byte but was measured slower; RT = 1 is what runs.
#include "linear_thin.h"

#include <type_traits>

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

// The same product for up to 16 rows and a long K, as a stream: fewer blocks than strips, each walking over
// its strips (strip = block, block + grid, ...) with the weight reads of the next steps always in flight, also
// across the end of a strip.  A wave keeps a ring of U super-steps: it uses the oldest and at once asks for
// the one U ahead into the same registers, so the memory pipe never drains between a block's first and last
// byte; only the last U steps of a block ask for nothing.  With TREG > 0 a wave's share of the activations
// (super-steps wave, wave + NW, ..., TREG of them, the same for every strip) is read once and stays in
// registers; with TREG == 0 it is read again beside every weight read: an activation read costs
// the cache path as much as a weight read although it brings nothing new.
// T: steps a wave makes for one strip, a multiple of U; steps beyond K read the row's start and count as zeros
// (EXACT says there are none, and then nothing is checked).
// NW: waves a block.  This kernel runs with 4, for a K of fewer than 32 super-steps, which eight waves would share
// out badly (K = 2560: 20 super-steps are 3 steps for each of eight waves with 12 of 32 turns idle, but 5 for each of
// four); from 32 super-steps on the stream is linear_ring.hip's, eight waves a block, whose weights cross LDS.
// Few strips and a long K (an output projection: 256 strips) leave most of the chip without work.  Then K is
// cut into `parts` ranges, blockIdx.y names the range, and the block writes its partial sums to plane
// blockIdx.y of a [parts, M, N] float32 result; whoever reads the result adds the planes in their order (the
// norm that follows adds them to the residual stream), so the sum is the same bits every time.
//
// The norm around a product can be folded into it (RowNorm, linear_thin.h), which saves the norm's own kernel in a
// decode step.

// Waves that run at once in the usual launch: 8 on each of 256 compute units, one block of eight waves each.  Two
// blocks a unit (4096) were the rule once: measured at 8 rows, the gated product of 24576 x 4096 38.2 us against 36.6
// and the head of 151936 rows 216 against 214 (a decode step of 36 layers 4.04 against 3.99 ms); anything between
// (2560, 3072) leaves some units with twice the work of others and is much slower (4.58 ms).
constexpr int STREAM_WAVE_SLOTS = 2048;
constexpr int STREAM_WAVE_SLOTS_CUT = 6144; // with K cut into ranges a block's work is short: 24 waves a unit

template <int NW, int U, int TREG, bool EXACT, typename TC, int EPI>
__global__ __launch_bounds__(NW * WAVE) void linear_stream_kernel(const bf16_t* __restrict__ A,
                                                                  const bf16_t* __restrict__ W,
                                                                  TC* __restrict__ C, int M, int N, int K,
                                                                  int n_strips, int T_given, RowNorm norm) {
    // this block's range of K starts at super-step blockIdx.y * T * NW, its results go to plane blockIdx.y
    constexpr bool AREG = TREG > 0;
    constexpr int PER = NW * 4;                  // threads that share a row's sum of squares
    static_assert(NW == 4 || NW == 8, "the epilogues count on 256 or 512 threads");
    __shared__ float part[2][NW][16][17];
    __shared__ float row_factor[16];
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    const int r = lane % 16, g = lane / 16;
    const int inter = N / 2;
    const int T = AREG ? TREG : T_given;
    const int first_super = blockIdx.y * T * NW;
    if (EPI == EPI_STORE) C += (size_t)blockIdx.y * M * N;

    auto row_of = [&](int strip) -> const bf16_t* {
        int wrow;
        if (EPI == EPI_SWIGLU) wrow = (r < 8 ? 0 : inter) + min(strip * 8 + (r % 8), inter - 1);
        else wrow = min(strip * 16 + r, N - 1);
        return W + (size_t)wrow * K + g * 8;
    };
    const bf16_t* xp = A + (size_t)min(r, M - 1) * K + g * 8;

    // the read cursor runs U steps ahead of the arithmetic
    int ask_strip = blockIdx.x, ask_t = 0;
    const bf16_t* ask_row = row_of(ask_strip);
    bf16x8 wv[U][4], xv[U][4];
    int present[U];                                          // bit j: chunk j of the slot lies inside K
    auto ask = [&](int u) {
        const int k0 = (first_super + ask_t * NW + wave) * SUPER_K;
        int mask = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bool ok = EXACT || (k0 + j * 32 + g * 8 < K);
            const int at = ok ? k0 + j * 32 : 0;             // an absent chunk reads the row's start and is masked
            wv[u][j] = load_bf16x8(ask_row + at);
            if (!AREG) xv[u][j] = load_bf16x8(xp + at);
            mask |= (ok ? 1 : 0) << j;
        }
        present[u] = mask;
        if (++ask_t == T) {
            ask_t = 0;
            ask_strip += gridDim.x;
            ask_row = row_of(min(ask_strip, n_strips - 1));
        }
    };
#pragma unroll
    for (int u = 0; u < U; ++u) ask(u);                      // weights first: they come from furthest away

    bf16x8 xa[AREG ? TREG : 1][4];
    if (AREG) {
#pragma unroll
        for (int t = 0; t < TREG; ++t) {
            const int k0 = (first_super + t * NW + wave) * SUPER_K;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bool ok = EXACT || (k0 + j * 32 + g * 8 < K);
                const bf16x8 v = load_bf16x8(xp + (ok ? k0 + j * 32 : 0));
                xa[t][j] = ok ? v : zero_bf16x8();
            }
        }
    }

    __builtin_amdgcn_sched_barrier(0);       // the weight reads above go out first, whatever follows
    // The rows' factors: PER threads a row add up the pieces, every block in the same order.  The reads go out
    // here and are used only when the first strip's products are done, so nothing waits for them.
    const int f_col = min((int)threadIdx.x / PER, M - 1), f_piece = threadIdx.x % PER;
    float piece[8];
    if (norm.ss_in) {
#pragma unroll
        for (int u = 0; u < 8; ++u)
            piece[u] = norm.ss_in[(size_t)f_col * norm.pieces_in + min(f_piece + PER * u, norm.pieces_in - 1)];
    }
    auto publish_row_factors = [&]() {
        float sum = 0.f;
#pragma unroll
        for (int u = 0; u < 8; ++u) sum += f_piece + PER * u < norm.pieces_in ? piece[u] : 0.f;
        for (int p = PER * 8 + f_piece; p < norm.pieces_in; p += PER) sum += norm.ss_in[(size_t)f_col * norm.pieces_in + p];
#pragma unroll
        for (int off = PER / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off, WAVE);
        if (f_piece == 0) row_factor[threadIdx.x / PER] = 1.0f / sqrtf(sum / (float)norm.width_in + norm.eps_in);
    };

    int buf = 0;
    for (int strip = blockIdx.x; strip < n_strips; strip += gridDim.x) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        const bool last = strip + (int)gridDim.x >= n_strips;
        // the residual element this thread will add to, asked for before the strip's products
        float x_old = 0.f, w_next = 0.f;
        if (EPI == EPI_STORE && norm.resid && threadIdx.x < 256) {
            const int feat = strip * 16 + threadIdx.x % 16, col = threadIdx.x / 16;
            if (col < M && feat < N) {
                x_old = norm.resid[(size_t)col * N + feat];
                w_next = norm.w_out[feat];
            }
        }
        // U steps: use each slot and, if `refill`, ask for the step U ahead into it
        auto steps = [&](int t, auto refill) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    bf16x8 wj = wv[u][j];
                    bf16x8 xj = AREG ? xa[AREG && t + u < TREG ? t + u : 0][j] : xv[u][j];
                    // a chunk beyond K counts as zeros: it is enough that the activations do (held in registers they
                    // were zeroed when read); the weights read in their place are the row's first, finite if any are
                    if (!EXACT && !AREG) xj = ((present[u] >> j) & 1) ? xj : zero_bf16x8();
                    acc = mfma_16x16x32(wj, xj, acc);
                }
                if (decltype(refill)::value) ask(u);
            }
        };
        if (AREG) {
#pragma unroll
            for (int t = 0; t + U < TREG; t += U) steps(t, std::true_type{});
            if (last) steps(TREG - U, std::false_type{});
            else steps(TREG - U, std::true_type{});
        } else {
            for (int t = 0; t + U < T; t += U) steps(0, std::true_type{});
            if (last) steps(0, std::false_type{});
            else steps(0, std::true_type{});
        }

        // partial tiles of the waves are added in a fixed order; two buffers, so one barrier a strip is enough
#pragma unroll
        for (int i = 0; i < 4; ++i) part[buf][wave][4 * g + i][r] = acc[i];
        if (norm.ss_in && strip == (int)blockIdx.x) publish_row_factors();
        __syncthreads();
        if (EPI == EPI_SWIGLU) {
            if (threadIdx.x < 128) {
                const int c = threadIdx.x % 8, col = threadIdx.x / 8;
                float gate = 0.f, up = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w) { gate += part[buf][w][c][col]; up += part[buf][w][c + 8][col]; }
                if (norm.ss_in) { gate *= row_factor[col]; up *= row_factor[col]; }
                const int feat = strip * 8 + c;
                if (col < M && feat < inter) C[(size_t)col * inter + feat] = from_float<TC>(gate / (1.0f + expf(-gate)) * up);
            }
        } else {
            if (threadIdx.x < 256) {
                const int row = threadIdx.x % 16, col = threadIdx.x / 16;
                float v = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w) v += part[buf][w][row][col];
                if (norm.ss_in) v *= row_factor[col];
                const int feat = strip * 16 + row;
                const bool mine = col < M && feat < N;
                if (norm.resid) {
                    const float x_new = x_old + v;
                    if (mine) {
                        norm.resid[(size_t)col * N + feat] = x_new;
                        C[(size_t)col * N + feat] = from_float<TC>(x_new * w_next);
                    }
                    float sq = mine ? x_new * x_new : 0.f;          // the 16 features of a row sit in 16 lanes side by side
#pragma unroll
                    for (int off = 8; off > 0; off >>= 1) sq += __shfl_xor(sq, off, WAVE);
                    if (row == 0 && col < M) norm.ss_out[(size_t)col * n_strips + strip] = sq;
                } else if (mine) {
                    C[(size_t)col * N + feat] = from_float<TC>(v);
                }
            }
        }
        buf ^= 1;
    }
}

// waves a block: eight, or four when K has fewer than 32 super-steps
static int stream_waves(int n_super) { return n_super < 32 ? 4 : 8; }

// steps a wave makes for one strip when K is cut into `parts` ranges
static int stream_steps(int n_super, int parts) {
    const int per_part = (n_super + parts - 1) / parts;
    const int nw = stream_waves(n_super);
    return (per_part + nw - 1) / nw;
}

// The steps the kernel variants make for a wish of `steps`: 2, 4, 6 or 8 with the activations in registers
// (K up to 8192), else a multiple of 4 with the activations read beside the weights, which for more than a few
// rows is much the slower way (2 against 5 TB/s at 16 rows).
constexpr int STREAM_MAX_REG_STEPS = 8;
static int stream_steps_served(int steps) { return steps <= STREAM_MAX_REG_STEPS ? (steps + 1) / 2 * 2 : (steps + 3) / 4 * 4; }

// Into how many ranges K is best cut for an [M, K] x [N, K]^T product whose reader can add planes: enough
// to give every compute unit two or three blocks, no fewer than two steps for a wave, and no range empty.
static int stream_parts(int M, int N, int K) {
    const int n_super = (K + SUPER_K - 1) / SUPER_K;
    if (M > 16 || n_super < 16) return 1;
    const int nw = stream_waves(n_super);
    const int strips = (N + 15) / 16;
    int parts = max(1, min(min(768 / strips, n_super / (2 * nw)), 4));
    // and enough to let a wave keep its share of the activations in registers
    parts = max(parts, min(4, (n_super + STREAM_MAX_REG_STEPS * nw - 1) / (STREAM_MAX_REG_STEPS * nw)));
    for (;;) {      // rounding the steps up can leave the last ranges without work: fewer ranges then
        const int covered = stream_steps_served(stream_steps(n_super, parts)) * nw;
        const int needed = (n_super + covered - 1) / covered;
        if (needed == parts) return parts;
        parts = needed;
    }
}

template <int NW, int U, int TREG, typename TC, int EPI>
static void launch_stream(hipStream_t stream, const void* a, const void* w, void* c, int M, int N, int K, int parts,
                          const RowNorm& norm) {
    const int strips = EPI == EPI_SWIGLU ? (N / 2 + 7) / 8 : (N + 15) / 16;
    const int n_super = (K + SUPER_K - 1) / SUPER_K;
    int T = stream_steps(n_super, parts);
    T = (T + U - 1) / U * U;
    if (TREG > 0) T = TREG;
    // every block the same number of strips, as far as that goes
    // (with six or eight steps of activations in registers more waves than the usual do not fit a compute unit)
    const int wave_slots = parts > 1 && TREG <= 4 ? STREAM_WAVE_SLOTS_CUT : STREAM_WAVE_SLOTS;
    const int slots = max(1, wave_slots / NW / parts);
    const int rounds = (strips + slots - 1) / slots;
    const dim3 grid((strips + rounds - 1) / rounds, parts);
    if (K % SUPER_K == 0 && parts * T * NW == n_super)
        linear_stream_kernel<NW, U, TREG, true, TC, EPI><<<grid, NW * WAVE, 0, stream>>>(
            (const bf16_t*)a, (const bf16_t*)w, (TC*)c, M, N, K, strips, T, norm);
    else
        linear_stream_kernel<NW, U, TREG, false, TC, EPI><<<grid, NW * WAVE, 0, stream>>>(
            (const bf16_t*)a, (const bf16_t*)w, (TC*)c, M, N, K, strips, T, norm);
}

template <int NW, typename TC, int EPI>
static void dispatch_stream(hipStream_t stream, const void* a, const void* w, void* c, int M, int N, int K, int parts,
                            const RowNorm& norm, int per_wave) {
    if (per_wave <= 2) launch_stream<NW, 2, 2, TC, EPI>(stream, a, w, c, M, N, K, parts, norm);
    else if (per_wave <= 4) launch_stream<NW, 2, 4, TC, EPI>(stream, a, w, c, M, N, K, parts, norm);
    else if (per_wave <= 6) launch_stream<NW, 2, 6, TC, EPI>(stream, a, w, c, M, N, K, parts, norm);
    else if (per_wave <= 8) launch_stream<NW, 2, 8, TC, EPI>(stream, a, w, c, M, N, K, parts, norm);
    else launch_stream<NW, 4, 0, TC, EPI>(stream, a, w, c, M, N, K, parts, norm);
}

template <typename TC, int EPI>
static void dispatch_thin(hipStream_t stream, const void* a, const void* w, void* c, int M, int N, int K, int parts,
                          const RowNorm& norm) {
    const int n_super = (K + SUPER_K - 1) / SUPER_K;
    const bool deep = n_super >= 16;                           // enough super-steps to feed a block's waves
    const bool folded = norm.ss_in || norm.resid;              // only the stream kernel folds a norm in
    if (M <= 16 && (deep || folded)) {
        const int per_wave = stream_steps(n_super, parts);
        // eight waves: the stream whose weights cross LDS; four (a short K): the one that reads them into registers
        if (stream_waves(n_super) == 8)
            launch_linear_ring(stream, a, w, c, sizeof(TC) == 2 ? PALM_BF16 : PALM_F32, M, N, K, EPI, parts, per_wave, norm);
        else
            dispatch_stream<4, TC, EPI>(stream, a, w, c, M, N, K, parts, norm, per_wave);
        return;
    }
    // a short K: one strip a block, four waves (two strips a block, RT = 2, were measured slower at every size)
    launch_thin<1, 4, 2, 1, TC, EPI>(stream, a, w, c, M, N, K);
}

PALM_API int palm_linear_thin_parts(int M, int N, int K) { return stream_parts(M, N, K); }

// a [M, K] bfloat16, w [N, K] bfloat16; c [M, N] (EPI_STORE) or [M, N/2] (EPI_SWIGLU) in bfloat16 or float32.
// parts > 1 (at most palm_linear_thin_parts(M, N, K), float32, EPI_STORE): c is [parts, M, N] and the product is
// the sum of its planes.
// ss_in (with pieces_in, eps_in, width_in = K) and resid (with w_out, ss_out) fold a norm in, see RowNorm; both
// need M <= 16, resid needs EPI_STORE, parts == 1 and a bfloat16 c, which then holds the next activations.
PALM_API int palm_linear_thin(hipStream_t stream, const void* a, const void* w, void* c, int c_dtype, int M, int N,
                              int K, int epilogue, int parts, const float* ss_in, int pieces_in, float eps_in,
                              float* resid, const float* w_out, float* ss_out) {
    PALM_CHECK(parts >= 1, "linear_thin: parts = %d", parts);
    RowNorm norm{ss_in, pieces_in, eps_in, K, resid, w_out, ss_out};
    PALM_CHECK(!(ss_in || resid) || M <= 16, "linear_thin: a norm is folded in for at most 16 rows, not %d", M);
    PALM_CHECK(!ss_in || pieces_in > 0, "linear_thin: %d pieces of the rows' sums of squares", pieces_in);
    PALM_CHECK(!resid || (epilogue == EPI_STORE && parts == 1 && c_dtype == PALM_BF16 && w_out && ss_out),
               "linear_thin: adding to the residual stream needs a plain bfloat16 product in one plane, the next norm's "
               "weight and room for the sums of squares");
    PALM_CHECK(parts == 1 || (epilogue == EPI_STORE && c_dtype == PALM_F32 && parts <= stream_parts(M, N, K)),
               "linear_thin: %d partial planes are not served for M=%d N=%d K=%d, this epilogue and result type", parts, M, N, K);
    PALM_CHECK(M >= 0 && N > 0 && K > 0, "linear_thin: M=%d N=%d K=%d", M, N, K);
    PALM_CHECK(K % 8 == 0, "linear_thin: K = %d is not a multiple of 8 (rows must start on 16 bytes)", K);
    // a lane's place among a strip's rows, in the activations and in the residual stream is a 32-bit byte offset
    PALM_CHECK((double)17 * K * 2 < 4.0e9 && (double)16 * N * 4 < 4.0e9, "linear_thin: N=%d K=%d is beyond 32-bit offsets", N, K);
    PALM_CHECK(epilogue == EPI_STORE || epilogue == EPI_SWIGLU, "linear_thin: epilogue %d", epilogue);
    PALM_CHECK(epilogue != EPI_SWIGLU || N % 2 == 0, "linear_thin: a gated product needs an even N, got %d", N);
    PALM_CHECK(((uintptr_t)a | (uintptr_t)w) % 16 == 0, "linear_thin: operands must be 16-byte aligned");
    if (M == 0) return 0;
    PALM_CHECK(M <= 16, "linear_thin: %d rows are more than the 16 of one block of tokens (linear_wide takes up to 64)", M);
    if (epilogue == EPI_SWIGLU) {
        PALM_DTYPE_SWITCH(c_dtype, TC, dispatch_thin<TC, EPI_SWIGLU>(stream, a, w, c, M, N, K, 1, norm));
    } else {
        PALM_DTYPE_SWITCH(c_dtype, TC, dispatch_thin<TC, EPI_STORE>(stream, a, w, c, M, N, K, parts, norm));
    }
    PALM_LAUNCHED();
    return 0;
}
