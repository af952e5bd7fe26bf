// C[M, N] = A[M, K] . W[N, K]^T for 33 to some hundred rows (decode steps of many sequences, short prompts): bfloat16
// on the matrix cores, 32-bit accumulation.  Too many rows for a wave to keep a strip of weights against all of them in
// registers, too few for the tiles of thousands of rows that a BLAS library is tuned for: the weights (some tens to
// hundreds of MB) pass once, from HBM, and must not wait; the rows (up to a few MB) are read again by every block,
// from L2.
//
// A block of four waves owns R rows (64, 128 or 256: all of them, for up to 256; more rows are more blocks beside it,
// numbered so that the blocks that share weights run on one die at about the same time) and TN weight rows (128, 96
// or 64: the most that still gives every compute unit a block), and a range of K (cut in up to four where the weight
// rows are few; the ranges' partial sums are float32 planes that the reader adds, as for the other kernels).  K goes
// by in chunks of 64.  Both operands of a chunk go from memory straight into LDS (global_load_lds: no registers, no
// write instruction, and every instruction brings eight whole 128-byte lines, which is what the vector cache takes
// at its full rate), each through a ring of its own: three chunks of rows (8 to 32 KB each; they come from L2), five
// chunks of weights (8 to 16 KB each; they come from HBM and need the longer lead), up to 156 KB of the 160 KB a
// compute unit has.  Every lane's loads are the same on every pass of the loop (beyond the range's end the last chunk
// is asked for once more, into a slot nobody reads any more), so the wait for "this chunk has landed" is a constant
// number of younger loads, and the compiler, which does not see the loads (they are written in assembly), adds no
// wait of its own.
//
// A wave multiplies its rows (64 of 256, 32 of 128, or 32 of 64 against half of the weight rows) with the block's
// weight rows: MFMA 32x32x16 with the weights as the first operand, so that a lane ends up with four neighbouring
// features of one token, which leave in one store; up to 2 x 3 tiles of 32 x 32, 96 accumulator registers.  One
// barrier a chunk, placed before the chunk's last step of k: the first fragments of the next chunk are then read from
// LDS while that step's matrix instructions run.  Rows of LDS are 128 bytes, their eight 16-byte pieces permuted by
// the row's number so that the lanes LDS serves together hit different banks.
// With the gated epilogue (out = silu(gate) * up, engine/cuda_ops.cu:100-112) a tile of 32 weight rows is sixteen
// gate rows and the sixteen up rows that belong to them, which one lane then holds side by side.
#include "mfma.h"

typedef float f32x16 __attribute__((ext_vector_type(16)));

enum MidEpilogue : int { MID_STORE = 0, MID_SWIGLU = 1 };

constexpr int MID_MAX_ROWS = 256;               // rows of A a block holds: 64, 128 or 256
constexpr int MID_WAVES = 4;
constexpr int MID_THREADS = MID_WAVES * WAVE;
constexpr int MID_CHUNK = 64;                   // k-values a step: a row of LDS is 128 bytes
constexpr int MID_ROW_BYTES = MID_CHUNK * 2;
constexpr int MID_MAX_STAGES = 4;    // (a decode step of 64 sequences: 8.04 ms with three, 7.83 with four, 7.87 with five, 7.90 with six)
constexpr int MID_LDS_BYTES = 160 * 1024;
constexpr int MID_MAX_PARTS = 4;
constexpr int MID_UNITS = 256;                  // compute units of the chip

// 16 bytes a lane from memory into LDS, the 64 lanes' pieces side by side from lds_base on.  base is the same in every
// lane (scalar registers), offset the lane's own.
__device__ __forceinline__ void mid_load_16_bytes_a_lane_into_lds(const void* base, uint32_t offset, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(offset), "s"(base), "s"(lds_base) : "m0", "memory");
}
template <int N> __device__ __forceinline__ void mid_wait_for_all_but_the_youngest_loads() {
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));          // s_waitcnt vmcnt(N)
}
// all but the youngest `groups` groups of LOADS loads each (at most three groups)
template <int LOADS> __device__ __forceinline__ void mid_wait_for_all_but_groups(int groups) {
    static_assert(3 * LOADS < 64, "the counter has six bits");
    if (groups >= 3) mid_wait_for_all_but_the_youngest_loads<3 * LOADS>();
    else if (groups == 2) mid_wait_for_all_but_the_youngest_loads<2 * LOADS>();
    else if (groups == 1) mid_wait_for_all_but_the_youngest_loads<1 * LOADS>();
    else mid_wait_for_all_but_the_youngest_loads<0>();
}
__device__ __forceinline__ void mid_barrier() {        // LDS reads done, then the block's barrier; loads stay in flight
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
__device__ __forceinline__ uint32_t mid_lds_address(const void* p) {
    return __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p);
}
__device__ inline f32x16 mfma_32x32x16(bf16x8 a, bf16x8 b, f32x16 acc) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
}

// R: rows of A a block holds.  TN: weight rows it holds (a multiple of 32; of 64 for 64 rows).  TC: element type of the
// result.  With 256 rows a wave has 64 of them (two tiles of 32) against all weight rows, with 128 rows 32 of them;
// with 64 rows a wave has 32 rows against half of the weight rows.
template <int R, int TN, typename TC, int EPI>
__global__ __launch_bounds__(MID_THREADS) void linear_mid_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, TC* __restrict__ C, int M, int N, int K,
    int n_tiles, int m_tiles, int chunks_per_part, int turn_blocks) {
    constexpr int NT = TN / 32;                                 // tiles of 32 weight rows
    constexpr int MT = R == 256 ? 2 : 1;                        // tiles of 32 rows a wave holds
    constexpr int NTW = R == 64 ? NT / 2 : NT;                  // tiles of weight rows a wave holds
    static_assert(R == 64 || R == 128 || R == 256, "a block holds 64, 128 or 256 rows");
    static_assert(R != 64 || NT % 2 == 0, "with 64 rows the waves share the weight tiles in halves");
    constexpr int MID_A_BYTES = R * MID_ROW_BYTES;              // a chunk of rows: 8, 16 or 32 KB
    constexpr int MID_A_LOADS = MID_A_BYTES / 1024 / MID_WAVES; // a wave's instructions for it: 2, 4 or 8
    constexpr int W_BYTES = TN * MID_ROW_BYTES;
    constexpr int W_LOADS = W_BYTES / 1024 / MID_WAVES;         // a wave's instructions for a chunk of weights
    static_assert(W_BYTES % (1024 * MID_WAVES) == 0, "a chunk of weights is a whole number of instructions a wave");
    // The rings.  All loads come back in the order they went out, and one counter counts them all: a wait for the rows
    // of the next chunk is also a wait for every load asked for before them.  So what is still on its way after a
    // pass's wait is what was asked for after the younger of the next chunk's two operands, and the rings are as deep
    // in flight as the shallower of them.  With 64 or 128 rows both rings have the same depth, four chunks (64 rows x
    // 128 weight rows: 4 x 24 KB, of which two are on their way after a wait).  256 rows leave room for three chunks
    // of rows and five of weights.
    constexpr bool SAME = R != 256;
    constexpr int BOTH = (MID_LDS_BYTES / (MID_A_BYTES + W_BYTES)) < MID_MAX_STAGES ? (MID_LDS_BYTES / (MID_A_BYTES + W_BYTES)) : MID_MAX_STAGES;
    constexpr int A_STAGES = SAME ? BOTH : 3;
    constexpr int W_STAGES = SAME ? BOTH : (MID_LDS_BYTES - 3 * MID_A_BYTES) / W_BYTES < 5 ? (MID_LDS_BYTES - 3 * MID_A_BYTES) / W_BYTES : 5;
    // loads asked for after the chunk that is due, see the loop
    constexpr int YOUNGER = SAME ? (A_STAGES - 2) * (MID_A_LOADS + W_LOADS) : W_LOADS + MID_A_LOADS + W_LOADS;
    constexpr int YOUNGER_AT_START = SAME ? (A_STAGES - 1) * (MID_A_LOADS + W_LOADS) : (W_STAGES - 1) * W_LOADS + 2 * MID_A_LOADS;
    static_assert(A_STAGES >= 3 && W_STAGES >= 3 && A_STAGES <= 4 + (SAME ? 0 : 8) && YOUNGER_AT_START < 64, "the rings' depth and the counter's six bits");
    __shared__ __attribute__((aligned(1024))) char a_lds[A_STAGES * MID_A_BYTES];
    __shared__ __attribute__((aligned(1024))) char w_lds[W_STAGES * W_BYTES];

    const int lane = threadIdx.x % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    // blocks 8 apart run on one die: they are the row tiles of one tile of weights, which so passes through that
    // die's L2 once; then the next tile of weights (or range of K)
    const int linear = blockIdx.x;
    const int group = linear / (8 * m_tiles), within = linear % (8 * m_tiles);
    const int m_tile = within / 8;
    const int work = group * 8 + within % 8;                    // (tile of weights, range of K)
    const int n_tile = work % n_tiles, part = work / n_tiles;
    const int inter = N / 2;
    const int features = EPI == MID_SWIGLU ? inter : N;
    const int f0 = n_tile * (EPI == MID_SWIGLU ? TN / 2 : TN);  // the block's first output feature
    if (f0 >= features) return;                                 // (the launch is padded to whole groups of eight)
    const int row0 = m_tile * R;
    const int n_chunks = K / MID_CHUNK;
    const int c0 = part * chunks_per_part, c1 = min(n_chunks, c0 + chunks_per_part);
    if (c0 >= c1) return;
    if (EPI == MID_STORE && sizeof(TC) == 4) C += (size_t)part * M * N;        // planes of partial sums

    // A lane's place in an instruction's kilobyte: row (its instruction's first row + lane / 8), piece lane % 8 of LDS,
    // which holds the row's piece (lane % 8) ^ (row % 8).  Rows beyond the last read the last (and are not stored).
    uint32_t a_from[MID_A_LOADS], w_from[W_LOADS];
#pragma unroll
    for (int i = 0; i < MID_A_LOADS; ++i) {
        const int row = (wave * MID_A_LOADS + i) * 8 + lane / 8;
        const int piece = (lane % 8) ^ (row % 8);
        a_from[i] = (uint32_t)min(row0 + row, M - 1) * (uint32_t)K * 2u + piece * 16;
    }
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i) {
        const int row = (wave * W_LOADS + i) * 8 + lane / 8;   // of the block's TN
        const int piece = (lane % 8) ^ (row % 8);
        int feature;
        if (EPI == MID_SWIGLU) {        // a tile of 32: sixteen gate rows, then their up rows
            const int f = min(f0 + (row / 32) * 16 + row % 16, inter - 1);
            feature = (row % 32 < 16 ? 0 : inter) + f;
        } else {
            feature = min(f0 + row, N - 1);
        }
        w_from[i] = (uint32_t)feature * (uint32_t)K * 2u + piece * 16;
    }
    const uint32_t a_lds0 = mid_lds_address(a_lds), w_lds0 = mid_lds_address(w_lds);
    // Where a block begins in its range of K.  Weight rows are K elements apart, a power of two in most models, and
    // blocks that walk over K in step ask the memory for the same few hundred bytes of every row at the same time:
    // the same few channels.  Where K is not cut (many weight rows: the gated product, the head) tile b of the weights begins b
    // chunks into K and wraps around, which spreads the blocks over the channels: the head for 64 rows 283 to 231 us,
    // gate/up for 128 rows 52 to 47.  Where K is cut the rows' share of the traffic is larger, and blocks out of step
    // no longer find each other's rows in L2 (down projection for 128 rows 33 to 38 us; with only the dies out of step
    // with each other nothing changes): those keep step.
    const int turn = turn_blocks ? work % (c1 - c0) : 0;       // (the row tiles of one tile of weights keep step)
    auto turned = [&](int chunk) __attribute__((always_inline)) { const int t = chunk - c0 + turn; return c0 + (t >= c1 - c0 ? t - (c1 - c0) : t); };
    // beyond the range's end: its last chunk once more, into a slot that nobody reads any more
    auto ask_rows = [&](int chunk) __attribute__((always_inline)) {
        const char* base = reinterpret_cast<const char*>(A) + (size_t)turned(min(chunk, c1 - 1)) * MID_ROW_BYTES;
        const uint32_t to = a_lds0 + ((chunk - c0) % A_STAGES) * MID_A_BYTES + wave * MID_A_LOADS * 1024;
#pragma unroll
        for (int i = 0; i < MID_A_LOADS; ++i) mid_load_16_bytes_a_lane_into_lds(base, a_from[i], to + i * 1024);
    };
    auto ask_weights = [&](int chunk) __attribute__((always_inline)) {
        const char* base = reinterpret_cast<const char*>(W) + (size_t)turned(min(chunk, c1 - 1)) * MID_ROW_BYTES;
        const uint32_t to = w_lds0 + ((chunk - c0) % W_STAGES) * W_BYTES + wave * W_LOADS * 1024;
#pragma unroll
        for (int i = 0; i < W_LOADS; ++i) mid_load_16_bytes_a_lane_into_lds(base, w_from[i], to + i * 1024);
    };

    // fragments: lane l holds row l % 32 of a tile and the eight k-values 16 s + 8 (l / 32) .. of step s
    const int fr = lane % 32, fh = lane / 32;
    const int wave_row0 = R == 256 ? wave * 64 : R == 128 ? wave * 32 : (wave % 2) * 32;     // the wave's first row
    const int wave_tile0 = R == 64 ? (wave / 2) * NTW : 0;                                  // and its first weight tile
    struct Fragments { bf16x8 w[NTW], x[MT]; };
    auto read = [&](int a_stage, int w_stage, int step, Fragments& f) __attribute__((always_inline)) {
        const char* wp = w_lds + w_stage * W_BYTES;
        const char* xp = a_lds + a_stage * MID_A_BYTES;
        const int piece = 2 * step + fh;
#pragma unroll
        for (int t = 0; t < NTW; ++t) {
            const int row = (wave_tile0 + t) * 32 + fr;
            f.w[t] = *reinterpret_cast<const bf16x8*>(wp + row * MID_ROW_BYTES + ((piece ^ (row % 8)) * 16));
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int row = wave_row0 + mt * 32 + fr;
            f.x[mt] = *reinterpret_cast<const bf16x8*>(xp + row * MID_ROW_BYTES + ((piece ^ (row % 8)) * 16));
        }
    };
    f32x16 acc[NTW][MT];
#pragma unroll
    for (int t = 0; t < NTW; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[t][mt][i] = 0.f;
    auto products = [&](const Fragments& f) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < NTW; ++t)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[t][mt] = mfma_32x32x16(f.w[t], f.x[mt], acc[t][mt]);
    };

    // The rings fill.  Pass c of the loop asks for the rows of chunk c + A_STAGES and then the weights of chunk
    // c + W_STAGES, and waits, before that, for chunk c + 1 with all that was asked for after the younger of its
    // operands still on its way.  The loads go out here in the order in which the passes before the first would have
    // asked for them, so that the first pass finds them as every later pass does.  Rings of the same depth: rows and
    // weights of a chunk side by side.  Three chunks of rows and more of weights: the weights asked for in the pass of
    // the next chunk's rows, and the rows and weights of the pass after, come last.
    if (SAME) {
        // (a short range asks for no chunk beyond its end, and the waits count what was asked for)
#pragma unroll
        for (int s = 0; s < A_STAGES; ++s)
            if (c0 + s < c1) { ask_rows(c0 + s); ask_weights(c0 + s); }
        mid_wait_for_all_but_groups<MID_A_LOADS + W_LOADS>(min(A_STAGES, c1 - c0) - 1);
    } else {
        ask_rows(c0);
#pragma unroll
        for (int s = 0; s < W_STAGES - 2; ++s) ask_weights(c0 + s);
        ask_rows(c0 + 1);
        ask_weights(c0 + W_STAGES - 2);
        ask_rows(c0 + 2);
        ask_weights(c0 + W_STAGES - 1);
        mid_wait_for_all_but_the_youngest_loads<YOUNGER_AT_START>();      // the first chunk's rows and weights are there
    }
    mid_barrier();
    Fragments f[2];
    read(0, 0, 0, f[0]);
    for (int c = c0; c < c1; ++c) {
        const int a_stage = (c - c0) % A_STAGES, w_stage = (c - c0) % W_STAGES;
#pragma unroll
        for (int step = 0; step < MID_CHUNK / 16 - 1; ++step) {
            read(a_stage, w_stage, step + 1, f[(step + 1) & 1]);
            products(f[step & 1]);
        }
        // The chunk's last fragments are in registers (or on their way: the barrier waits for them).  The next chunk
        // must have landed, for every wave's share of it: all but the loads asked for after it are done.
        if (SAME) {
            // after chunk c + 1 come the chunks up to c + A_STAGES - 1, as far as the range goes; at its end nothing
            // is asked for any more, and the last passes wait for fewer
            mid_wait_for_all_but_groups<MID_A_LOADS + W_LOADS>(min(A_STAGES - 2, c1 - 2 - c));
            mid_barrier();
            if (c + A_STAGES < c1) { ask_rows(c + A_STAGES); ask_weights(c + A_STAGES); }       // into the slots this chunk's readers have left
        } else {
            mid_wait_for_all_but_the_youngest_loads<YOUNGER>();
            mid_barrier();
            ask_rows(c + A_STAGES);                             // into the slots that this chunk's readers have left
            ask_weights(c + W_STAGES);
        }
        if (c + 1 < c1) read((c + 1 - c0) % A_STAGES, (c + 1 - c0) % W_STAGES, 0, f[0]);
        products(f[(MID_CHUNK / 16 - 1) & 1]);
    }
    mid_wait_for_all_but_the_youngest_loads<0>();               // nothing of this block is on its way when it ends

    // lane l holds token column l % 32 of each tile and, of the tile's 32 weight rows, rows 8 j + 4 (l / 32) + 0..3 as
    // elements 4 j .. 4 j + 3
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int token = row0 + wave_row0 + mt * 32 + fr;
        if (token >= M) continue;
#pragma unroll
        for (int t = 0; t < NTW; ++t) {
            if (EPI == MID_SWIGLU) {
                // rows 0..15 of the tile are gate rows, 16..31 their up rows: elements 4 j + i and 4 (j + 2) + i
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int feature = f0 + (wave_tile0 + t) * 16 + 8 * j + 4 * fh;
                    float out[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float gate = acc[t][mt][4 * j + i], up = acc[t][mt][4 * (j + 2) + i];
                        out[i] = gate / (1.0f + expf(-gate)) * up;
                    }
                    TC* to = C + (size_t)token * inter + feature;
                    if (feature + 3 < inter && inter % 4 == 0) {
                        if constexpr (sizeof(TC) == 2) {
                            uint2 four;
                            four.x = (uint32_t)f32_to_bf16(out[0]).bits | ((uint32_t)f32_to_bf16(out[1]).bits << 16);
                            four.y = (uint32_t)f32_to_bf16(out[2]).bits | ((uint32_t)f32_to_bf16(out[3]).bits << 16);
                            *reinterpret_cast<uint2*>(to) = four;
                        } else {
                            *reinterpret_cast<float4*>(to) = make_float4(out[0], out[1], out[2], out[3]);
                        }
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i) if (feature + i < inter) to[i] = from_float<TC>(out[i]);
                    }
                }
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int feature = f0 + (wave_tile0 + t) * 32 + 8 * j + 4 * fh;
                    const float out[4] = {acc[t][mt][4 * j], acc[t][mt][4 * j + 1], acc[t][mt][4 * j + 2], acc[t][mt][4 * j + 3]};
                    TC* to = C + (size_t)token * N + feature;
                    if (feature + 3 < N && N % 4 == 0) {
                        if constexpr (sizeof(TC) == 2) {
                            uint2 four;
                            four.x = (uint32_t)f32_to_bf16(out[0]).bits | ((uint32_t)f32_to_bf16(out[1]).bits << 16);
                            four.y = (uint32_t)f32_to_bf16(out[2]).bits | ((uint32_t)f32_to_bf16(out[3]).bits << 16);
                            *reinterpret_cast<uint2*>(to) = four;
                        } else {
                            *reinterpret_cast<float4*>(to) = make_float4(out[0], out[1], out[2], out[3]);
                        }
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i) if (feature + i < N) to[i] = from_float<TC>(out[i]);
                    }
                }
            }
        }
    }
}

struct MidPlan { int rows, tn, parts, chunks_per_part, n_tiles, m_tiles; };

// rows a block holds for a product of M rows
static int mid_rows(int M) { return M <= 64 ? 64 : M <= 128 ? 128 : MID_MAX_ROWS; }

// Weight rows a block (128, 96 or 64: what fits LDS beside the rows, and with 64 rows an even number of tiles) and
// ranges of K: what takes the fewest rounds of blocks over the compute units, a round costing its chunks (and a few
// for filling the rings) times the block's weight rows.
static MidPlan mid_plan(int M, int N, int K, int epilogue, int max_parts) {
    const int n_chunks = K / MID_CHUNK;
    const int rows = mid_rows(M);
    const int m_tiles = (M + rows - 1) / rows;
    MidPlan best{rows, 64, 1, n_chunks, 1, m_tiles};
    long best_cost = -1;
    for (int tn = 128; tn >= 64; tn -= 32) {
        if ((rows == 256 && tn == 128) || (rows == 64 && tn == 96)) continue;
        const int per_block = epilogue == MID_SWIGLU ? tn / 2 : tn;
        const int features = epilogue == MID_SWIGLU ? N / 2 : N;
        const int n_tiles = (features + per_block - 1) / per_block;
        for (int parts = 1; parts <= max_parts; ++parts) {
            const int per = (n_chunks + parts - 1) / parts;
            if (parts > 1 && (per < 8 || (parts - 1) * per >= n_chunks)) continue;       // short, or an empty range
            const long blocks = (long)n_tiles * parts * m_tiles;
            const long cost = ((blocks + MID_UNITS - 1) / MID_UNITS) * (per + 6) * tn;
            if (best_cost < 0 || cost < best_cost) { best_cost = cost; best = MidPlan{rows, tn, parts, per, n_tiles, m_tiles}; }
        }
    }
    return best;
}

// Into how many planes the product comes if the caller takes planes (1: the result itself).
PALM_API int palm_linear_mid_parts(int M, int N, int K, int epilogue) {
    if (epilogue == MID_SWIGLU || M <= 0 || N <= 0 || K < MID_CHUNK) return 1;
    return mid_plan(M, N, K, epilogue, MID_MAX_PARTS).parts;
}

// How many blocks the launch would have: a caller with another way to the product takes that when these are few.
PALM_API int palm_linear_mid_blocks(int M, int N, int K, int epilogue, int planes_ok) {
    if (M <= 0 || N <= 0 || K < MID_CHUNK) return 0;
    const MidPlan plan = mid_plan(M, N, K, epilogue, planes_ok && epilogue == MID_STORE ? MID_MAX_PARTS : 1);
    return plan.n_tiles * plan.parts * plan.m_tiles;
}

template <int R, int TN, typename TC, int EPI>
static void launch_mid(hipStream_t stream, const void* a, const void* w, void* c, int M, int N, int K, MidPlan plan) {
    const int work = plan.n_tiles * plan.parts;
    const int groups = (work + 7) / 8;                          // whole groups of eight tiles of weights, a die each
    linear_mid_kernel<R, TN, TC, EPI><<<groups * 8 * plan.m_tiles, MID_THREADS, 0, stream>>>(
        (const bf16_t*)a, (const bf16_t*)w, (TC*)c, M, N, K, plan.n_tiles, plan.m_tiles, plan.chunks_per_part,
        plan.parts == 1 ? 1 : 0);
}

template <int R, int TN>
static void launch_mid_as(hipStream_t stream, const void* a, const void* w, void* c, int c_dtype, int M, int N, int K,
                          int epilogue, MidPlan plan) {
    if (epilogue == MID_SWIGLU) launch_mid<R, TN, bf16_t, MID_SWIGLU>(stream, a, w, c, M, N, K, plan);
    else if (c_dtype == PALM_BF16) launch_mid<R, TN, bf16_t, MID_STORE>(stream, a, w, c, M, N, K, plan);
    else launch_mid<R, TN, float, MID_STORE>(stream, a, w, c, M, N, K, plan);
}

// a [M, K] bfloat16, w [N, K] bfloat16, K a multiple of 64; c [M, N] (store) or [M, N/2] (gated) in bfloat16, or, with
// parts > 1 (as palm_linear_mid_parts says; store only), float32 planes [parts, M, N]; parts == 1 with c_dtype float32
// is one float32 plane, the result itself.
PALM_API int palm_linear_mid(hipStream_t stream, const void* a, const void* w, void* c, int c_dtype, int M, int N, int K,
                             int epilogue, int parts) {
    PALM_CHECK(M >= 0 && N > 0 && K > 0, "linear_mid: M=%d N=%d K=%d", M, N, K);
    PALM_CHECK(K % MID_CHUNK == 0, "linear_mid: K = %d is not a multiple of %d", K, MID_CHUNK);
    PALM_CHECK(epilogue == MID_STORE || epilogue == MID_SWIGLU, "linear_mid: epilogue %d", epilogue);
    PALM_CHECK(epilogue != MID_SWIGLU || N % 2 == 0, "linear_mid: a gated product needs an even N, got %d", N);
    PALM_CHECK(((uintptr_t)a | (uintptr_t)w | (uintptr_t)c) % 16 == 0, "linear_mid: operands must be 16-byte aligned");
    PALM_CHECK(c_dtype == PALM_BF16 || c_dtype == PALM_F32, "linear_mid: result type %d", c_dtype);
    // a lane's place in the rows and in the weights is a 32-bit byte offset
    PALM_CHECK((double)M * K * 2 < 4.0e9 && (double)N * K * 2 < 4.0e9, "linear_mid: M=%d N=%d K=%d is beyond 32-bit offsets", M, N, K);
    const MidPlan plan = mid_plan(M, N, K, epilogue, parts > 1 ? MID_MAX_PARTS : 1);
    PALM_CHECK(parts == 1 || (parts == plan.parts && epilogue == MID_STORE && c_dtype == PALM_F32),
               "linear_mid: %d planes asked for, %d planned (planes are float32, not gated)", parts, plan.parts);
    PALM_CHECK(epilogue == MID_STORE || c_dtype == PALM_BF16, "linear_mid: a gated product comes in bfloat16");
    if (M == 0) return 0;
#define PALM_MID(R, TN) launch_mid_as<R, TN>(stream, a, w, c, c_dtype, M, N, K, epilogue, plan)
    if (plan.rows == 64) { if (plan.tn == 128) PALM_MID(64, 128); else PALM_MID(64, 64); }
    else if (plan.rows == 128) { if (plan.tn == 128) PALM_MID(128, 128); else if (plan.tn == 96) PALM_MID(128, 96); else PALM_MID(128, 64); }
    else { if (plan.tn == 96) PALM_MID(256, 96); else PALM_MID(256, 64); }
#undef PALM_MID
    PALM_LAUNCHED();
    return 0;
}
