// C[M, N] = A[M, K] . W[N, K]^T for 17 to 128 rows (decode steps of large batches, short prompts): bfloat16 on the matrix
// cores, 32-bit accumulation.  The thin kernels (linear_mfma.hip) let every wave fetch the activations it
// needs straight from the caches, which for more than 16 rows is several times the weight traffic; here a
// block shares them through LDS.
//
// A block has NW waves (4, 6 or 8, chosen with the number of K ranges so that the launch fills the compute
// units evenly), each with a strip of 16 weight rows of its own against all MB*16 rows of A, and one range of
// K (grid.y; the ranges' partial results are float32 planes [parts, M, N] that the reader adds up in the order
// of the planes, as the norm after a projection and the q/k/v pass do).  K goes by in chunks of 256 (of 128 for more
// than 64 rows, whose operands would else not fit the registers and LDS).  A lane's
// reads are a ring of three or four slots; a slot holds the eight weight fragments of one chunk (64 contiguous bytes
// of a row per instruction, as in the thin kernels) and the lane's share of the activations of the chunk
// after it.  Reads come back in the order they went out, so the wait for a slot leaves the younger slots
// in flight: activations never make a wave wait for weights that it asked for later.  When a slot is due, its
// weights meet the activations that lie in LDS since the step before (two buffers, one barrier a chunk; rows
// padded by 16 bytes, so that the lanes LDS serves together hit different banks), its activations go into the other buffer, and the slot asks for the chunk a ring's length on.
// With the gated epilogue (out = silu(gate) * up, engine/cuda_ops.cu:100-112) a wave's strip is eight gate
// rows and the eight up rows that belong to them.
#pragma once
#include "mfma.h"

#include <type_traits>

enum WideEpilogue : int { WIDE_STORE = 0, WIDE_SWIGLU = 1 };

// k-values a step, by the blocks of 16 rows a launch holds
__host__ __device__ constexpr int wide_chunk(int row_blocks) { return row_blocks <= 4 ? 256 : 128; }
// Slots of reads: a slot is 8 KB of weights a wave; the slot in use is not in flight, and a compute unit wants about
// 100 KB on their way; four slots where the registers hold them (one wave a SIMD, or 32 rows), else three
__host__ __device__ constexpr int wide_ring(int waves, int row_blocks) { return waves <= 4 || row_blocks <= 2 ? 4 : 3; }
constexpr int WIDE_MAX_ROWS = 128;
constexpr int WIDE_MAX_PARTS = 4;               // as many planes as the readers of planes add up
constexpr int WIDE_MIN_CHUNKS = 4;              // a range of K is not shorter than this
constexpr int WIDE_UNITS = 256;                 // compute units of the chip: a launch comes in rounds of so many blocks

// four results side by side in one store (the address is a multiple of the store's size)
__device__ inline void store4(float* to, const float (&v)[4]) { *reinterpret_cast<float4*>(to) = make_float4(v[0], v[1], v[2], v[3]); }
__device__ inline void store4(bf16_t* to, const float (&v)[4]) {
    uint2 four;
    four.x = (uint32_t)f32_to_bf16(v[0]).bits | ((uint32_t)f32_to_bf16(v[1]).bits << 16);
    four.y = (uint32_t)f32_to_bf16(v[2]).bits | ((uint32_t)f32_to_bf16(v[3]).bits << 16);
    *reinterpret_cast<uint2*>(to) = four;
}

// f(integral_constant<int, 0>{}) ... f(integral_constant<int, N - 1>{}), in this order
template <typename F, int... I>
__device__ __forceinline__ void static_for_each(F&& f, std::integer_sequence<int, I...>) { (f(std::integral_constant<int, I>{}), ...); }
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) { static_for_each(f, std::make_integer_sequence<int, N>{}); }

// base is the same for all lanes, bytes a lane's own 32 bits, plus a constant: the three parts of a read's address
template <int PLUS = 0>
__device__ inline bf16x8 load_bf16x8_at(const char* base, uint32_t bytes) {
    return *reinterpret_cast<const bf16x8*>(base + (size_t)bytes + PLUS);
}

// EXACT: K is a multiple of the chunk, so no read is beyond K and none needs a condition.
template <int MB, int NW, bool EXACT, typename TC, int EPI>
__global__ __launch_bounds__(NW * WAVE) void linear_wide_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, TC* __restrict__ C, int M, int N, int K,
    int chunks_per_part) {
    constexpr int ROWS = MB * 16;
    constexpr int WIDE_CHUNK = wide_chunk(MB);                            // k-values a step
    constexpr int WIDE_PIECES = WIDE_CHUNK / 8;                           // 16-byte pieces of a row of the chunk
    constexpr int WIDE_STRIDE = WIDE_CHUNK + 8;                           // a row in LDS, padded: the 16 rows that lanes read together start in 16 different banks
    constexpr int FRAGMENTS = WIDE_CHUNK / 32;                            // matrix-core steps of a chunk
    constexpr int RING = wide_ring(NW, MB);
    constexpr int THREADS = NW * WAVE;
    constexpr int XS = (ROWS * WIDE_PIECES + THREADS - 1) / THREADS;      // pieces of a chunk's activations a thread carries
    constexpr int ROW_STEP = THREADS / WIDE_PIECES;                       // from one of a thread's pieces to its next: so many rows on
    constexpr int STRIP_ROWS = EPI == WIDE_SWIGLU ? 8 : 16;               // output features of a strip
    constexpr uint32_t CHUNK_BYTES = WIDE_CHUNK * sizeof(bf16_t);
    __shared__ __attribute__((aligned(16))) bf16_t x_lds[2][ROWS * WIDE_STRIDE];
    const int lane = threadIdx.x % WAVE, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int r = lane % 16, g = lane / 16;
    const int inter = N / 2;
    const int features = EPI == WIDE_SWIGLU ? inter : N;

    // The weight rows a wave reads start at w_base, the same for all its lanes, so that it and a chunk's step live
    // in scalar registers; a lane adds its row and k-group as 32 bits.  A strip beyond the last reads the last
    // strip's rows and drops its results; rows beyond the last feature read the last feature's.
    const int strip = blockIdx.x * NW + wave;
    const int first = min(strip, (features + STRIP_ROWS - 1) / STRIP_ROWS - 1) * STRIP_ROWS;
    const char* w_base = reinterpret_cast<const char*>(W + (size_t)first * K);
    const int w_row = (EPI == WIDE_SWIGLU && r >= 8 ? inter : 0) + min(r % STRIP_ROWS, features - 1 - first);
    const uint32_t w_lane = ((uint32_t)w_row * K + g * 8) * sizeof(bf16_t);

    const int n_chunks = (K + WIDE_CHUNK - 1) / WIDE_CHUNK;
    const int c0 = blockIdx.y * chunks_per_part, c1 = min(n_chunks, c0 + chunks_per_part);
    if (c0 >= c1) return;                      // (the host plans no empty range)
    if (gridDim.y > 1) C += (size_t)blockIdx.y * M * N;
    // Where a block begins in K.  Weight rows are K elements apart, a power of two in most models, and blocks that
    // walk over K in step ask the memory for the same few hundred bytes of every row at the same time: the same few
    // channels.  Where K is not cut and all blocks run at once (the gated product) block b begins b chunks into K
    // and wraps around: 44 to 40 us for 32 rows.  Where K is cut the blocks keep step: the rows' share of the traffic
    // is larger there, and blocks out of step no longer find each other's rows in L2.  Where the blocks come in
    // several rounds (the head) they are out of step by themselves, and turning them made it slower (252 to 279 us).
    const int turn = gridDim.y == 1 && gridDim.x <= WIDE_UNITS ? (int)(blockIdx.x % (unsigned)(c1 - c0)) : 0;
    auto turned = [&](int chunk) __attribute__((always_inline)) { const int t = chunk - c0 + turn; return c0 + (t >= c1 - c0 ? t - (c1 - c0) : t); };

    f32x4 acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};

    // This thread's pieces of a chunk's activations: piece x_piece of rows x_row0, x_row0 + ROW_STEP, ...
    const int x_row0 = threadIdx.x / WIDE_PIECES, x_piece = threadIdx.x % WIDE_PIECES;
    auto row_live = [&](int i) __attribute__((always_inline)) { return x_row0 + i * ROW_STEP < min(M, ROWS); };
    const char* x_base = reinterpret_cast<const char*>(A);
    uint32_t x_row[XS];                        // where the rows start, in bytes
#pragma unroll
    for (int i = 0; i < XS; ++i) x_row[i] = (uint32_t)min(x_row0 + i * ROW_STEP, M - 1) * K * sizeof(bf16_t);

    bf16x8 wf[RING][FRAGMENTS], xs[RING][XS];
    auto ask_rows = [&](int logical, auto slot) __attribute__((always_inline)) {
        constexpr int s = decltype(slot)::value;
        const int chunk = turned(logical);
        // what lies beyond M or K reads a place that exists; put_rows makes zeros of it
        const bool ok = EXACT || chunk * WIDE_CHUNK + x_piece * 8 < K;
        const char* from = x_base + (ok ? chunk * CHUNK_BYTES : 0);
        const uint32_t at = ok ? x_piece * 16 : 0;
#pragma unroll
        for (int i = 0; i < XS; ++i) xs[s][i] = load_bf16x8_at(from, x_row[i] + at);
    };
    auto ask_weights = [&](int logical, auto slot) __attribute__((always_inline)) {
        constexpr int s = decltype(slot)::value;
        const int chunk = turned(logical);
        const char* from = w_base + (size_t)chunk * CHUNK_BYTES;
        static_for<FRAGMENTS>([&](auto jc) __attribute__((always_inline)) {
            constexpr int j = decltype(jc)::value;
            if (EXACT) {
                wf[s][j] = load_bf16x8_at<j * 64>(from, w_lane);
            } else {        // beyond K: the row's start is read; the activations there are zeros
                const bool ok = chunk * WIDE_CHUNK + j * 32 + g * 8 < K;
                wf[s][j] = load_bf16x8_at(ok ? from : w_base, ok ? w_lane + j * 64 : w_lane - g * 16);
            }
        });
    };
    auto put_rows = [&](int buf, int logical, auto slot) __attribute__((always_inline)) {
        constexpr int s = decltype(slot)::value;
        const int chunk = turned(logical);
        const bool in_k = EXACT || chunk * WIDE_CHUNK + x_piece * 8 < K;
#pragma unroll
        for (int i = 0; i < XS; ++i) {
            const int row = x_row0 + i * ROW_STEP;
            if (row < ROWS)
                *reinterpret_cast<bf16x8*>(&x_lds[buf][row * WIDE_STRIDE + x_piece * 8]) =
                    in_k && row_live(i) ? xs[s][i] : zero_bf16x8();
        }
    };
    // a chunk's products, the B operands read from LDS one group of k ahead of their use
    auto products = [&](int buf, auto slot) __attribute__((always_inline)) {
        constexpr int s = decltype(slot)::value;
        bf16x8 xf[2][MB];
        auto fetch = [&](int j, int into) __attribute__((always_inline)) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                const int row = mb * 16 + r, piece = j * 4 + g;
                xf[into][mb] = *reinterpret_cast<const bf16x8*>(&x_lds[buf][row * WIDE_STRIDE + piece * 8]);
            }
        };
        fetch(0, 0);
#pragma unroll
        for (int j = 0; j < FRAGMENTS; ++j) {
            if (j + 1 < FRAGMENTS) fetch(j + 1, (j + 1) & 1);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) acc[mb] = mfma_16x16x32(wf[s][j], xf[j & 1][mb], acc[mb]);
            __builtin_amdgcn_sched_barrier(0);             // or all 32 operands are fetched before the first product
        }
    };

    // Slot (c - c0) % RING holds the weights of chunk c and the activations of chunk c + 1.  Every read below is
    // issued on every path that reaches it (no read sits under a condition), so the compiler knows how many
    // younger reads a wait may leave in flight.  Where the range has no such chunk left, its last chunk is asked
    // for once more: it comes from the caches, nothing uses it, and no read leaves the matrices.
    auto fill = [&](int c, auto slot) __attribute__((always_inline)) {
        ask_rows(min(c + 1, c1 - 1), slot);
        ask_weights(min(c, c1 - 1), slot);
    };
    // the first chunk's activations borrow the last slot's registers; the slot is filled once they are in LDS,
    // which waits for them alone, the oldest reads
    using Last = std::integral_constant<int, RING - 1>;
    ask_rows(c0, Last{});
    static_for<RING - 1>([&](auto s) __attribute__((always_inline)) { fill(c0 + decltype(s)::value, s); });
    put_rows(0, c0, Last{});
    fill(c0 + RING - 1, Last{});
    __syncthreads();

    int buf = 0, c = c0;
    auto step = [&](auto slot, auto refill) __attribute__((always_inline)) {
        products(buf, slot);
        if (c + 1 < c1) put_rows(buf ^ 1, c + 1, slot);
        if (decltype(refill)::value) fill(c + RING, slot);
        __syncthreads();                                   // the other buffer is whole; this one is free again
        buf ^= 1;
        ++c;
    };
    // rounds in which every step has a chunk to ask for
    while (c + 2 * RING <= c1)
        static_for<RING>([&](auto s) __attribute__((always_inline)) { step(s, std::true_type{}); });
    // more than one round left: its first steps still have chunks to ask for; the others ask for the range's last
    // chunk once more (it comes from the caches and is not used), so that the round is the same code on every path
    if (c + RING < c1)
        static_for<RING>([&](auto s) __attribute__((always_inline)) { step(s, std::true_type{}); });
    // the ring runs dry
    static_for<RING>([&](auto s) __attribute__((always_inline)) { if (c < c1) step(s, std::false_type{}); });

    // this lane holds token column r of each block mb, weight rows 4g + i of the wave's strip
    if (EPI == WIDE_SWIGLU) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            const int tok = mb * 16 + r;
            float out[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float up = __shfl(acc[mb][i], (lane + 32) % WAVE, WAVE);     // row 4g + i + 8 lives 32 lanes on
                const float gate = acc[mb][i];
                out[i] = gate / (1.0f + expf(-gate)) * up;
            }
            const int feat = strip * 8 + 4 * g;
            if (g < 2 && tok < M) {
                TC* to = C + (size_t)tok * inter + feat;
                if (feat + 3 < inter && inter % 4 == 0) store4(to, out);
                else
#pragma unroll
                    for (int i = 0; i < 4; ++i) if (feat + i < inter) to[i] = from_float<TC>(out[i]);
            }
        }
    } else {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            const int tok = mb * 16 + r, feat = strip * 16 + 4 * g;
            if (tok >= M) continue;
            TC* to = C + (size_t)tok * N + feat;
            const float out[4] = {acc[mb][0], acc[mb][1], acc[mb][2], acc[mb][3]};
            if (feat + 3 < N && N % 4 == 0) store4(to, out);
            else
#pragma unroll
                for (int i = 0; i < 4; ++i) if (feat + i < N) to[i] = from_float<TC>(out[i]);
        }
    }
}

struct WidePlan { int waves, parts, chunks_per_part; };

template <int MB, int NW, typename TC, int EPI>
static void launch_wide(hipStream_t stream, const void* a, const void* w, void* c, int M, int N, int K, WidePlan plan) {
    const int strips = EPI == WIDE_SWIGLU ? (N / 2 + 7) / 8 : (N + 15) / 16;
    dim3 grid((strips + NW - 1) / NW, plan.parts);
    if (K % wide_chunk(MB) == 0)
        linear_wide_kernel<MB, NW, true, TC, EPI><<<grid, NW * WAVE, 0, stream>>>(
            (const bf16_t*)a, (const bf16_t*)w, (TC*)c, M, N, K, plan.chunks_per_part);
    else
        linear_wide_kernel<MB, NW, false, TC, EPI><<<grid, NW * WAVE, 0, stream>>>(
            (const bf16_t*)a, (const bf16_t*)w, (TC*)c, M, N, K, plan.chunks_per_part);
}

template <int MB, typename TC, int EPI>
static void launch_wide_waves(hipStream_t stream, const void* a, const void* w, void* c, int M, int N, int K, WidePlan plan) {
    if (plan.waves == 4) launch_wide<MB, 4, TC, EPI>(stream, a, w, c, M, N, K, plan);
    else if (plan.waves == 6) launch_wide<MB, 6, TC, EPI>(stream, a, w, c, M, N, K, plan);
    else launch_wide<MB, 8, TC, EPI>(stream, a, w, c, M, N, K, plan);
}

// The kernels are instantiated in six files (store or gated epilogue; 32, 64 or 128 rows), which compile side by side.
void wide_launch_store_32(hipStream_t stream, const void* a, const void* w, void* c, int c_dtype, int M, int N, int K, WidePlan plan);
void wide_launch_store_64(hipStream_t stream, const void* a, const void* w, void* c, int c_dtype, int M, int N, int K, WidePlan plan);
void wide_launch_gated_32(hipStream_t stream, const void* a, const void* w, void* c, int c_dtype, int M, int N, int K, WidePlan plan);
void wide_launch_gated_64(hipStream_t stream, const void* a, const void* w, void* c, int c_dtype, int M, int N, int K, WidePlan plan);
void wide_launch_store_128(hipStream_t stream, const void* a, const void* w, void* c, int c_dtype, int M, int N, int K, WidePlan plan);
void wide_launch_gated_128(hipStream_t stream, const void* a, const void* w, void* c, int c_dtype, int M, int N, int K, WidePlan plan);

#define PALM_WIDE_INSTANCE(NAME, MB, EPI) \
    void NAME(hipStream_t stream, const void* a, const void* w, void* c, int c_dtype, int M, int N, int K, WidePlan plan) { \
        if (c_dtype == PALM_BF16) launch_wide_waves<MB, bf16_t, EPI>(stream, a, w, c, M, N, K, plan); \
        else launch_wide_waves<MB, float, EPI>(stream, a, w, c, M, N, K, plan); \
    }
