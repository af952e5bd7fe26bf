// C[M, N] = X[M, K] . W[N, K]^T for many rows: bfloat16 operands on the matrix cores, 32-bit accumulation.  The
// product is the reference's matmul (kernels/matmul_dense.cpp:939-953), which its GPU path hands to a library
// (engine/cuda_matmul.cu:245-260), and so does this engine for a prompt's products.  This kernel is here for what
// that library call cannot give: a float32 result from bfloat16 operands, the logits at many places of a prompt.
// (It once had epilogues that applied the gated activation or added the product to the residual stream; for many
// rows the library's kernel with a pass of its own after it was the faster way, and they are gone.)
//
// Tiling.  A block of eight waves owns TOK tokens x FEAT features and walks over K (or, with K cut into ranges, over
// its range) in stages of 64.  A stage of both operands lies in LDS as rows of 128 bytes (64 k-values: a whole
// cache line; stages of 32 were measured slower, half of every line fetched being of no use to the stage), features
// first, then tokens, in a ring of as many stages as LDS holds (two of 256 + 256 rows, three of 256 + 128).  Rows
// go from memory straight into LDS (global_load_lds, 16 bytes a lane, an instruction fills 1 KB = 8 rows); a row's
// eight 16-byte chunks are permuted by the row number (chunk ^ ((row >> 1) & 7)) so that the 16-byte reads of a
// matrix instruction's operand, consecutive rows at the same k, spread over the banks.  The lane that fills a place
// fetches the chunk that belongs there, so the permutation costs nothing.
// What bounds it: a compute unit reads at most some 45 GB/s of what its die's L2 does not hold (measured with the
// products and the LDS reads taken out, through registers or straight into LDS, with one, two or three stages in
// flight; a long prompt's operands are far larger than L2), 11 to 12 TB/s for the chip; a tile of 256 x 256 needs 128 KB for every 64 k-values, which is 270 us for the gate/up product of
// 2,048 rows, about what the library's kernel of the same tile takes in all.  This kernel overlaps its products
// and its reads less well (360 us), so prompts keep the library; it serves where a library call cannot: float32
// results of many rows (logits at many places).
// MFMA 32x32x16: the A operand is 32 weight rows (features), the B operand 32 activation rows (tokens); a lane
// of the result holds one token and 16 features in runs of four, so results leave as 8-byte (bfloat16) or
// 16-byte (float32) pieces of a token's row.
// Waves: WAVES_F x WAVES_T = 8; a wave owns (FEAT / WAVES_F) x (TOK / WAVES_T) of the tile, NF x NT matrix
// tiles.  With two waves on a SIMD one wave's LDS reads hide behind the other's products.
//
// Blocks are numbered so that the 32 blocks that run on one die at a time (blocks go to the eight dies in turn)
// work on neighbouring tiles: each die's L2 then holds few weight and activation tiles for many blocks.
#include "mfma.h"

#ifdef PALM_TILE_STANDALONE
PALM_DEFINE_LAST_ERROR()
#endif

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int TK = 64;                       // k-values of a stage
constexpr int ROW_BYTES = TK * 2;            // a row of a stage in LDS
constexpr int ROW_CHUNKS = ROW_BYTES / 16;   // 16-byte chunks of such a row
constexpr int ROWS_AN_INSTRUCTION = 1024 / ROW_BYTES;
constexpr int SUB_STEPS = TK / 16;           // matrix instructions' k-steps in a stage
constexpr int LDS_BYTES = 160 * 1024;
constexpr int TILE_WAVES = 8;
constexpr int TILE_THREADS = TILE_WAVES * WAVE;
constexpr int DIES = 8;

__device__ __forceinline__ void row_chunk_into_lds(const void* from, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(from), "s"(lds_base) : "m0", "memory");
}
// s_waitcnt vmcnt(N): loads come back in order, so "all but the N youngest" is a stage's rows with the later stages'
// still on their way.  (vmcnt is six bits: the low four in bits 0..3, the high two in bits 14..15.)
template <int N> __device__ __forceinline__ void all_but_the_youngest_have_arrived() {
    static_assert(N >= 0 && N < 64, "vmcnt has six bits");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

template <int TOK, int FEAT, int WAVES_F, typename TC>
__global__ __launch_bounds__(TILE_THREADS) void linear_tile_kernel(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                                                                   TC* __restrict__ C, int M, int N, int K, int tiles_t,
                                                                   int tiles_f) {
    constexpr int WAVES_T = TILE_WAVES / WAVES_F;
    constexpr int NF = FEAT / WAVES_F / 32, NT = TOK / WAVES_T / 32;
    constexpr int ROWS = FEAT + TOK, STAGE = ROWS * ROW_BYTES, PER_WAVE = ROWS / ROWS_AN_INSTRUCTION / TILE_WAVES;
    constexpr int RING = (LDS_BYTES - 8 * 1024) / STAGE > 6 ? 6 : (LDS_BYTES - 8 * 1024) / STAGE;      // stages in LDS
    constexpr int AHEAD = RING - 1;                                                                      // of which on their way
    static_assert(FEAT % (32 * WAVES_F) == 0 && TOK % (32 * WAVES_T) == 0 && ROWS % (ROWS_AN_INSTRUCTION * TILE_WAVES) == 0,
                  "tile and waves do not fit");
    static_assert(RING >= 2 && (AHEAD - 1) * PER_WAVE < 64, "the ring does not fit LDS or the load counter");
    __shared__ __attribute__((aligned(1024))) char lds[RING * STAGE];

    // which tile: blocks pid, pid + 8, .. run on one die; give each die a run of neighbouring tiles
    const int total = tiles_t * tiles_f, per_die = (total + DIES - 1) / DIES;
    const int pid = (blockIdx.x % DIES) * per_die + blockIdx.x / DIES;
    if (pid >= total) return;
    // this block's range of K, in stages, and the plane its sums go to
    const int all_stages = K / TK, per_range = (all_stages + (int)gridDim.y - 1) / (int)gridDim.y;
    const int first_stage = blockIdx.y * per_range, stages = min(per_range, all_stages - first_stage);
    C += (size_t)blockIdx.y * M * N;
    const int tile_t = pid % tiles_t, tile_f = pid / tiles_t;       // the token tiles of a feature tile side by side
    const int t0 = tile_t * TOK;
    const int f0 = tile_f * FEAT;

    const int lane = threadIdx.x % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int wave_f = wave % WAVES_F, wave_t = wave / WAVES_F;

    // ---- the rows this lane brings in: instruction q of this wave fills LDS rows (q * 8 + wave) * 16 .. + 15
    const char* src[PER_WAVE];
#pragma unroll
    for (int q = 0; q < PER_WAVE; ++q) {
        const int R = (q * TILE_WAVES + wave) * ROWS_AN_INSTRUCTION + lane / ROW_CHUNKS;
        const int chunk = (lane % ROW_CHUNKS) ^ ((R >> 1) & (ROW_CHUNKS - 1));
        const bf16_t* row;
        if (R < FEAT) {
            row = W + (size_t)min(f0 + R, N - 1) * K;
        } else {
            row = X + (size_t)min(t0 + R - FEAT, M - 1) * K;
        }
        src[q] = reinterpret_cast<const char*>(row) + (size_t)first_stage * ROW_BYTES + chunk * 16;
    }
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)lds);
    auto bring = [&](int kt, int slot) {                       // stage kt of this block's range into a place of the ring
#pragma unroll
        for (int q = 0; q < PER_WAVE; ++q)
            row_chunk_into_lds(src[q] + (size_t)kt * ROW_BYTES, lds0 + slot * STAGE + (q * TILE_WAVES + wave) * 1024);
    };

    // ---- the operands this lane reads: rows of its matrix tiles, chunk 2 s + lane / 32 of sub-step s
    int w_off[NF], x_off[NT], cs[SUB_STEPS];
#pragma unroll
    for (int f = 0; f < NF; ++f) {
        w_off[f] = (wave_f * (FEAT / WAVES_F) + f * 32 + lane % 32) * ROW_BYTES;
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) x_off[t] = (FEAT + wave_t * (TOK / WAVES_T) + t * 32 + lane % 32) * ROW_BYTES;
#pragma unroll
    for (int s = 0; s < SUB_STEPS; ++s)         // every such row has (row >> 1) & 3 == (lane >> 1) & 3
        cs[s] = ((2 * s + lane / 32) ^ ((lane >> 1) & (ROW_CHUNKS - 1))) * 16;

    f32x16 acc[NF][NT];
#pragma unroll
    for (int f = 0; f < NF; ++f)
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[f][t][v] = 0.f;

    // The operands of sub-step s + 1 are read from LDS while the products of sub-step s run: a wave's own reads hide
    // behind its own products, and two waves on a SIMD fill what is left.
    auto read_operands = [&](const char* stage, int s, bf16x8 (&wf)[NF], bf16x8 (&xf)[NT]) {
#pragma unroll
        for (int f = 0; f < NF; ++f) wf[f] = *reinterpret_cast<const bf16x8*>(stage + w_off[f] + cs[s]);
#pragma unroll
        for (int t = 0; t < NT; ++t) xf[t] = *reinterpret_cast<const bf16x8*>(stage + x_off[t] + cs[s]);
    };
#pragma unroll
    for (int i = 0; i < AHEAD; ++i)
        if (i < stages) bring(i, i);
    int slot = 0;                                              // where stage kt lies in the ring
    for (int kt = 0; kt < stages; ++kt) {
        // stage kt has arrived when at most the AHEAD - 1 younger stages are still on their way; at the end of K
        // fewer are, and then everything is waited for
        if (kt + AHEAD <= stages) all_but_the_youngest_have_arrived<(AHEAD - 1) * PER_WAVE>();
        else all_but_the_youngest_have_arrived<0>();
        __syncthreads();                                       // every wave's share of it; and everyone is done with stage kt - 1
        if (kt + AHEAD < stages) bring(kt + AHEAD, slot == 0 ? RING - 1 : slot - 1);       // into the place of stage kt - 1
        const char* stage = lds + slot * STAGE;
        bf16x8 wf[2][NF], xf[2][NT];
        read_operands(stage, 0, wf[0], xf[0]);
#pragma unroll
        for (int s = 0; s < SUB_STEPS; ++s) {
            if (s + 1 < SUB_STEPS) read_operands(stage, s + 1, wf[(s + 1) & 1], xf[(s + 1) & 1]);
#pragma unroll
            for (int f = 0; f < NF; ++f)
#pragma unroll
                for (int t = 0; t < NT; ++t)
                    acc[f][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[s & 1][f], xf[s & 1][t], acc[f][t], 0, 0, 0);
            // the order asked of the compiler: a read of the next sub-step's operands after each of the first products
            if (s + 1 < SUB_STEPS) {
#pragma unroll
                for (int i = 0; i < NF + NT; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);      // one matrix instruction
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);      // one LDS read
                }
                __builtin_amdgcn_sched_group_barrier(0x008, NF * NT - NF - NT, 0);
            }
        }
        slot = slot + 1 == RING ? 0 : slot + 1;
    }

    // ---- epilogue.  Element v of a result tile: token lane % 32, feature 8 (v / 4) + 4 (lane / 32) + v % 4.
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int tok = t0 + wave_t * (TOK / WAVES_T) + t * 32 + lane % 32;
        if (tok >= M) continue;
#pragma unroll
        for (int f = 0; f < NF; ++f)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const int feat = f0 + wave_f * (FEAT / WAVES_F) + f * 32 + 8 * q4 + 4 * (lane / 32);
                if (feat >= N) continue;
                const float o[4] = {acc[f][t][4 * q4], acc[f][t][4 * q4 + 1], acc[f][t][4 * q4 + 2], acc[f][t][4 * q4 + 3]};
                TC* dst = C + (size_t)tok * N + feat;
                if (feat + 3 < N && N % 4 == 0) {
                    if constexpr (sizeof(TC) == 2) {
                        uint2 four;
                        four.x = (uint32_t)f32_to_bf16(o[0]).bits | ((uint32_t)f32_to_bf16(o[1]).bits << 16);
                        four.y = (uint32_t)f32_to_bf16(o[2]).bits | ((uint32_t)f32_to_bf16(o[3]).bits << 16);
                        *reinterpret_cast<uint2*>(dst) = four;
                    } else {
                        *reinterpret_cast<float4*>(dst) = make_float4(o[0], o[1], o[2], o[3]);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (feat + i < N) dst[i] = from_float<TC>(o[i]);
                }
            }
    }
}

// ---- launch -----------------------------------------------------------------------------------------
constexpr int TILE_FEAT = 256;

template <int TOK, int WAVES_F, typename TC>
static void launch_tile(hipStream_t stream, const void* x, const void* w, void* c, int M, int N, int K, int parts) {
    const int tiles_t = (M + TOK - 1) / TOK, tiles_f = (N + TILE_FEAT - 1) / TILE_FEAT;
    const int total = tiles_t * tiles_f, blocks = (total + DIES - 1) / DIES * DIES;
    linear_tile_kernel<TOK, TILE_FEAT, WAVES_F, TC><<<dim3(blocks, parts), TILE_THREADS, 0, stream>>>(
        (const bf16_t*)x, (const bf16_t*)w, (TC*)c, M, N, K, tiles_t, tiles_f);
}

// How many tokens a block takes: 256 where that still gives most compute units a block, else 128.
static int tile_tokens(int M, int N, int parts) {
    const int tiles_f = (N + TILE_FEAT - 1) / TILE_FEAT;
    if (M <= 128) return 128;
    return ((M + 255) / 256) * tiles_f * parts >= 192 ? 256 : 128;
}

// Into how many ranges K is cut when the reader takes float32 planes: enough to give most compute units a block,
// at most four, and no range shorter than 16 stages.
static int tile_parts(int M, int N, int K) {
    const int tiles = ((M + 127) / 128) * ((N + TILE_FEAT - 1) / TILE_FEAT);
    int parts = 1;
    while (parts < 4 && tiles * parts < 192 && K / TK / (parts + 1) >= 16) ++parts;
    return parts;
}
PALM_API int palm_linear_tile_parts(int M, int N, int K) { return tile_parts(M, N, K); }

template <typename TC>
static void dispatch_tile(hipStream_t stream, const void* x, const void* w, void* c, int M, int N, int K, int parts) {
    if (tile_tokens(M, N, parts) == 256) launch_tile<256, 2, TC>(stream, x, w, c, M, N, K, parts);
    else launch_tile<128, 4, TC>(stream, x, w, c, M, N, K, parts);
}

// x [M, K] bfloat16, w [N, K] bfloat16, K a multiple of 64; c [M, N] bfloat16 or float32; or, with parts > 1 (at most
// palm_linear_tile_parts(M, N, K)), float32 planes [parts, M, N], each the sum over one range of K, for a reader that
// adds them in their order.
PALM_API int palm_linear_tile(hipStream_t stream, const void* x, const void* w, void* c, int c_dtype, int M, int N, int K,
                              int parts) {
    PALM_CHECK(M >= 0 && N > 0 && K > 0, "linear_tile: M=%d N=%d K=%d", M, N, K);
    PALM_CHECK(K % TK == 0, "linear_tile: K = %d is not a multiple of %d", K, TK);
    PALM_CHECK(parts >= 1 && (parts == 1 || (c_dtype == PALM_F32 && parts <= 4 && K / TK >= parts)),
               "linear_tile: %d planes of partial sums (they are float32, at most four)", parts);
    PALM_CHECK(c_dtype == PALM_BF16 || c_dtype == PALM_F32, "linear_tile: result type %d", c_dtype);
    PALM_CHECK(((uintptr_t)x | (uintptr_t)w | (uintptr_t)c) % 16 == 0, "linear_tile: operands must be 16-byte aligned");
    PALM_CHECK((double)M * N < 2.0e9 * 4, "linear_tile: the result is beyond this kernel's index range");
    if (M == 0) return 0;
    PALM_DTYPE_SWITCH(c_dtype, TC, dispatch_tile<TC>(stream, x, w, c, M, N, K, parts));
    PALM_LAUNCHED();
    return 0;
}
