// C[M, N] = A[M, K] . W[N, K]^T for up to 16 rows and a long K (decode steps), the weights crossing LDS.
//
// The matrix instruction wants a lane to hold 16 bytes of weight row (lane % 16); a wave's read of that shape touches
// 16 cache lines 64 bytes at a time, and the vector cache takes such an instruction at a quarter of the rate of one
// whose eight neighbouring lanes share a line (measured with all compute units reading: 16 against 57 bytes a clock
// and unit; the stream of a decode step needs some 10).  So here no lane reads weights into registers.  A wave asks
// for a super-step (16 rows x 128 k-values, 4 KB) as four instructions that each bring eight whole 128-byte lines
// from memory straight into LDS (global_load_lds), into a ring of U slots of the wave's own, and reads the fragments
// for the matrix cores back from LDS; the 16-byte pieces of a line are permuted by the row's number on their way, so
// that the eight lanes LDS serves together hit different banks.  No registers carry data in flight, so the ring can
// be deep (four slots, 128 KB a compute unit on their way), and nothing of it is seen by the compiler: the waits are
// written here, as counts of the loads that may still be out (loads come back in the order they went; stores that are
// on their way only make such a wait stricter).
//
// Everything else is the stream kernel's (linear_mfma.hip): a block of eight waves owns whole strips of 16 weight rows
// (eight gate and their eight up rows with the gated epilogue, engine/cuda_ops.cu:100-112), walks over its strips with
// the reads running ahead across their ends, the waves take every eighth super-step and their partial tiles are
// added in LDS in a fixed order; K may be cut into ranges whose sums are float32 planes; a wave's share of the
// activations stays in registers where it fits (TREG super-steps), else it crosses LDS beside the weights; and the
// norm before and after the product can be folded in (RowNorm).
#include "linear_thin.h"

#include <type_traits>

constexpr int RING_WAVES = 8;
constexpr int RING_THREADS = RING_WAVES * WAVE;
constexpr int RING_UNITS = 256;                 // compute units: a launch is one block for each, or fewer

// 16 (4) bytes a lane from memory into LDS, the 64 lanes' pieces side by side from lds_base on.  base is the same in
// every lane (scalar registers), offset the lane's own.  LDS reads of the wave that are still out are waited for
// first: the slot that is asked for may be the one they read.
__device__ __forceinline__ void ring_load_16(const void* base, uint32_t offset, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(offset), "s"(base), "s"(lds_base) : "m0", "memory");
}
__device__ __forceinline__ void ring_load_4(const void* base, uint32_t offset, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" : : "v"(offset), "s"(base), "s"(lds_base) : "m0", "memory");
}
__device__ __forceinline__ void ring_lds_reads_done() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
template <int N> __device__ __forceinline__ void ring_wait_for_all_but_the_youngest_loads() {
    static_assert(N >= 0 && N < 64, "the counter has six bits");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));          // s_waitcnt vmcnt(N)
    asm volatile("" ::: "memory");
}
// all but the youngest `slots` slots of LOADS instructions each
template <int LOADS, int MAX> __device__ __forceinline__ void ring_wait_slots(int slots) {
    static_assert(MAX <= 4, "a ring of at most four slots");
    if (MAX >= 4 && slots >= 4) ring_wait_for_all_but_the_youngest_loads<4 * LOADS>();
    else if (MAX >= 3 && slots == 3) ring_wait_for_all_but_the_youngest_loads<3 * LOADS>();
    else if (MAX >= 2 && slots == 2) ring_wait_for_all_but_the_youngest_loads<2 * LOADS>();
    else if (MAX >= 1 && slots == 1) ring_wait_for_all_but_the_youngest_loads<1 * LOADS>();
    else ring_wait_for_all_but_the_youngest_loads<0>();
}
__device__ __forceinline__ void ring_barrier() {       // LDS traffic done, then the block's barrier; loads stay in flight
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
__device__ __forceinline__ uint32_t ring_lds_address(const void* p) {
    return __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p);
}

// U: slots of a wave's ring.  TREG: super-steps of activations a wave holds in registers (0: they cross LDS beside
// the weights).  T: steps a wave makes for one strip.  EXACT: no step is beyond K.
template <int U, int TREG, bool EXACT, typename TC, int EPI>
__global__ __launch_bounds__(RING_THREADS) void linear_ring_kernel(const bf16_t* __restrict__ A,
                                                                    const bf16_t* __restrict__ W,
                                                                    TC* __restrict__ C, int M, int N, int K,
                                                                    int n_strips, int T_given, RowNorm norm) {
    constexpr int NW = RING_WAVES;
    constexpr bool AREG = TREG > 0;
    constexpr int SLOT = AREG ? 4096 : 8192;                 // a super-step of weights, and of activations behind it
    constexpr int LOADS = SLOT / 1024;                       // instructions that fill a slot
    constexpr int PER = NW * 4;                              // threads that share a row's sum of squares
    constexpr int PIECES_HELD = 16;
    static_assert((U & (U - 1)) == 0 && U * LOADS < 64, "slots are counted modulo U, loads by a counter of six bits");
    __shared__ __attribute__((aligned(1024))) char ring[NW * U * SLOT];
    __shared__ float part[2][NW][16][17];
    __shared__ float row_factor[16];
    __shared__ float staged[2][RING_THREADS];                // the residual elements and norm weights of a strip
    const int lane = threadIdx.x % WAVE, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int r = lane % 16, g = lane / 16;
    const int inter = N / 2;
    const int T = AREG ? TREG : T_given;
    const int first_super = blockIdx.y * T * NW;
    if (EPI == EPI_STORE) C += (size_t)blockIdx.y * M * N;

    // What a lane asks for: in each of a slot's instructions, 16 bytes of row (lane / 8) of eight rows, piece
    // (lane % 8) ^ (lane / 8) of the line's eight; instruction i brings rows 8 (i % 2) .., k-values 64 (i / 2) ..
    const int row8 = lane / 8;
    const int piece = (lane % 8) ^ row8;
    // Where a strip's rows start (the same in every lane: scalar registers), its first eight and its second eight (with
    // the gated epilogue eight gate rows and the eight up rows that belong to them), and a lane's row among the eight
    // as a byte offset; rows beyond the last read the last.
    auto bases_of = [&](int strip, const char* (&base)[2]) __attribute__((always_inline)) {
        if (EPI == EPI_SWIGLU) {
            base[0] = reinterpret_cast<const char*>(W + (size_t)strip * 8 * K);
            base[1] = reinterpret_cast<const char*>(W + ((size_t)inter + (size_t)strip * 8) * K);
        } else {
            base[0] = reinterpret_cast<const char*>(W + (size_t)strip * 16 * K);
            base[1] = reinterpret_cast<const char*>(W + (size_t)min(strip * 16 + 8, N - 1) * K);
        }
    };
    auto rows_of = [&](int strip, uint32_t (&off)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            int rel;
            if (EPI == EPI_SWIGLU) rel = min(row8, inter - 1 - strip * 8);
            else rel = min(row8, max(0, N - 1 - min(strip * 16 + 8 * h, N - 1)));
            off[h] = (uint32_t)rel * (uint32_t)K * 2u;
        }
    };
    uint32_t x_off[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) x_off[h] = (uint32_t)min(h * 8 + row8, M - 1) * (uint32_t)K * 2u;
    // and where a lane finds its fragment of chunk j (32 k-values) in a slot: row r, pieces 4 (j % 2) + g of half j / 2
    uint32_t frag[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) frag[j] = ((r / 8) + 2 * (j / 2)) * 1024 + (r % 8) * 128 + ((((j % 2) * 4 + g) ^ (r % 8)) * 16);

    // the read cursor runs up to U steps ahead of the arithmetic, across the ends of strips
    const int my_strips = (n_strips - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
    const int total = my_strips * T;
    int n_asked = 0, n_used = 0;
    int ask_strip = blockIdx.x, ask_t = 0;
    const char* ask_base[2];
    uint32_t w_off[2];
    bases_of(ask_strip, ask_base);
    rows_of(ask_strip, w_off);
    const uint32_t ring0 = ring_lds_address(ring) + wave * (U * SLOT);
    auto ask = [&]() __attribute__((always_inline)) {
        const uint32_t to = ring0 + (n_asked & (U - 1)) * SLOT;
        const int k0 = (first_super + ask_t * NW + wave) * SUPER_K;
        ring_lds_reads_done();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            // K is a multiple of 8: a piece is whole or absent; an absent one reads the row's start and counts as zeros
            const bool ok = EXACT || k0 + (i / 2) * 64 + piece * 8 < K;
            const uint32_t in_row = ok ? (uint32_t)(k0 * 2 + (i / 2) * 128 + piece * 16) : 0u;
            ring_load_16(ask_base[i % 2], w_off[i % 2] + in_row, to + i * 1024);
            if (!AREG) ring_load_16(A, x_off[i % 2] + in_row, to + 4096 + i * 1024);
        }
        ++n_asked;
        if (++ask_t == T) {
            ask_t = 0;
            ask_strip += gridDim.x;
            const int s = min(ask_strip, n_strips - 1);
            bases_of(s, ask_base);
            rows_of(s, w_off);
        }
    };
    for (int u = 0; u < U && u < total; ++u) ask();          // weights first: they come from furthest away

    // A wave's share of the activations, read once; what lies beyond K is zeros, which makes the weights read in its
    // place (the row's first, finite if any are) count as nothing.
    bf16x8 xa[AREG ? TREG : 1][4];
    if (AREG) {
        const bf16_t* xp = A + (size_t)min(r, M - 1) * K + g * 8;
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
    // The rows' factors: PER threads a row add up the pieces, every block in the same order.
    const int f_col = min((int)threadIdx.x / PER, M - 1), f_piece = threadIdx.x % PER;
    float piece_ss[PIECES_HELD];
    if (norm.ss_in) {
#pragma unroll
        for (int u = 0; u < PIECES_HELD; ++u)
            piece_ss[u] = norm.ss_in[(size_t)f_col * norm.pieces_in + min(f_piece + PER * u, norm.pieces_in - 1)];
    }
    // These are the only reads the compiler knows of.  Its wait for them counts no load it does not know, so it would
    // also wait for whatever of the ring went out before that wait: it is made to stand here, where that is the
    // ring's first filling and nothing more.
    if (AREG) {
#pragma unroll
        for (int t = 0; t < TREG; ++t)
#pragma unroll
            for (int j = 0; j < 4; ++j) asm volatile("" : "+v"(xa[t][j]));
    }
    if (norm.ss_in) {
#pragma unroll
        for (int u = 0; u < PIECES_HELD; ++u) asm volatile("" : "+v"(piece_ss[u]));
    }
    auto publish_row_factors = [&]() {
        float sum = 0.f;
#pragma unroll
        for (int u = 0; u < PIECES_HELD; ++u) sum += f_piece + PER * u < norm.pieces_in ? piece_ss[u] : 0.f;
        for (int p = PER * PIECES_HELD + f_piece; p < norm.pieces_in; p += PER) sum += norm.ss_in[(size_t)f_col * norm.pieces_in + p];
#pragma unroll
        for (int off = PER / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off, WAVE);
        if (f_piece == 0) row_factor[threadIdx.x / PER] = 1.0f / sqrtf(sum / (float)norm.width_in + norm.eps_in);
    };

    // one step: the oldest slot has landed when all but the slots asked for after it have; its fragments meet the
    // activations; then the slot asks for the step U ahead
    auto step = [&](int t, f32x4& acc, const bf16x8 (&x)[4]) __attribute__((always_inline)) {
        ring_wait_slots<LOADS, U - 1>(min(U - 1, n_asked - n_used - 1));
        const char* slot = ring + (wave * U + (n_used & (U - 1))) * SLOT;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bf16x8 wj = *reinterpret_cast<const bf16x8*>(slot + frag[j]);
            bf16x8 xj;
            if (AREG) {
                xj = x[j];
            } else {
                xj = *reinterpret_cast<const bf16x8*>(slot + 4096 + frag[j]);
                const int k0 = (first_super + t * NW + wave) * SUPER_K;
                if (!EXACT && k0 + j * 32 + g * 8 >= K) xj = zero_bf16x8();
            }
            acc = mfma_16x16x32(wj, xj, acc);
        }
        ++n_used;
        if (n_asked < total) ask();
    };

    int buf = 0;
    for (int strip = blockIdx.x; strip < n_strips; strip += gridDim.x) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        // the residual elements the strip will be added to, and the next norm's weights: asked for before the strip's
        // products, through LDS like everything else (thread t and thread t + 256 ask for the same)
        const int asked_before = n_asked;
        if (EPI == EPI_STORE && norm.resid) {
            const int t256 = threadIdx.x % 256;
            const int feat = min(strip * 16 + t256 % 16, N - 1), col = min(t256 / 16, M - 1);
            ring_lds_reads_done();
            ring_load_4(norm.resid, (uint32_t)(col * N + feat) * 4u, ring_lds_address(&staged[0][0]) + wave * (WAVE * 4));
            ring_load_4(norm.w_out, (uint32_t)feat * 4u, ring_lds_address(&staged[1][0]) + wave * (WAVE * 4));
        }
        if (AREG) {
#pragma unroll
            for (int t = 0; t < TREG; ++t) step(t, acc, xa[t]);
        } else {
            for (int t = 0; t < T; ++t) step(t, acc, xa[0]);
        }

        // partial tiles of the waves are added in a fixed order; two buffers, so one barrier a strip is enough
#pragma unroll
        for (int i = 0; i < 4; ++i) part[buf][wave][4 * g + i][r] = acc[i];
        if (norm.ss_in && strip == (int)blockIdx.x) publish_row_factors();
        // what was staged at the strip's start is there when all but the slots asked for since then are
        if (EPI == EPI_STORE && norm.resid) ring_wait_slots<LOADS, U>(min(U, n_asked - asked_before));
        ring_barrier();
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
                    const float x_new = staged[0][threadIdx.x] + v;
                    if (mine) {
                        norm.resid[(size_t)col * N + feat] = x_new;
                        C[(size_t)col * N + feat] = from_float<TC>(x_new * staged[1][threadIdx.x]);
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

template <int U, int TREG, typename TC, int EPI>
static void launch_ring(hipStream_t stream, const void* a, const void* w, void* c, int M, int N, int K, int parts, int steps,
                        const RowNorm& norm) {
    const int strips = EPI == EPI_SWIGLU ? (N / 2 + 7) / 8 : (N + 15) / 16;
    const int n_super = (K + SUPER_K - 1) / SUPER_K;
    const int T = TREG > 0 ? TREG : steps;
    // one block a compute unit, every block the same number of strips, as far as that goes
    const int slots = max(1, RING_UNITS / parts);
    const int rounds = (strips + slots - 1) / slots;
    const dim3 grid((strips + rounds - 1) / rounds, parts);
    if (K % SUPER_K == 0 && parts * T * RING_WAVES == n_super)
        linear_ring_kernel<U, TREG, true, TC, EPI><<<grid, RING_THREADS, 0, stream>>>(
            (const bf16_t*)a, (const bf16_t*)w, (TC*)c, M, N, K, strips, T, norm);
    else
        linear_ring_kernel<U, TREG, false, TC, EPI><<<grid, RING_THREADS, 0, stream>>>(
            (const bf16_t*)a, (const bf16_t*)w, (TC*)c, M, N, K, strips, T, norm);
}

template <typename TC, int EPI>
static void dispatch_ring(hipStream_t stream, const void* a, const void* w, void* c, int M, int N, int K, int parts, int steps,
                          const RowNorm& norm) {
    if (steps <= 2) launch_ring<4, 2, TC, EPI>(stream, a, w, c, M, N, K, parts, steps, norm);
    else if (steps <= 4) launch_ring<4, 4, TC, EPI>(stream, a, w, c, M, N, K, parts, steps, norm);
    else if (steps <= 6) launch_ring<4, 6, TC, EPI>(stream, a, w, c, M, N, K, parts, steps, norm);
    else if (steps <= 8) launch_ring<4, 8, TC, EPI>(stream, a, w, c, M, N, K, parts, steps, norm);
    else launch_ring<2, 0, TC, EPI>(stream, a, w, c, M, N, K, parts, steps, norm);
}

void launch_linear_ring(hipStream_t stream, const void* a, const void* w, void* c, int c_dtype, int M, int N, int K,
                        int epilogue, int parts, int steps, const RowNorm& norm) {
    if (epilogue == EPI_SWIGLU) {
        if (c_dtype == PALM_BF16) dispatch_ring<bf16_t, EPI_SWIGLU>(stream, a, w, c, M, N, K, 1, steps, norm);
        else dispatch_ring<float, EPI_SWIGLU>(stream, a, w, c, M, N, K, 1, steps, norm);
    } else {
        if (c_dtype == PALM_BF16) dispatch_ring<bf16_t, EPI_STORE>(stream, a, w, c, M, N, K, parts, steps, norm);
        else dispatch_ring<float, EPI_STORE>(stream, a, w, c, M, N, K, parts, steps, norm);
    }
}
