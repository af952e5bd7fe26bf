// C[M, N] = X[M, K] . W[N, K]^T for many rows (prompts, decode steps of more than 64 sequences): bfloat16
// operands on the matrix cores, 32-bit accumulation.  The product is the reference's matmul
// (kernels/matmul_dense.cpp:939-953), which its GPU path hands to a library (engine/cuda_matmul.cu:245-260);
// this kernel is here for what a library call cannot do: an epilogue that applies the gated activation, or
// adds the product to the residual stream and prepares the next norm, so that neither [M, 2I] nor the branch
// output ever goes to memory, and tiles sized for some hundred rows, where the weight should go by once.
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
// results of many rows (logits at many places), and the epilogues below.
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

enum TileEpilogue : int { TILE_STORE = 0, TILE_SWIGLU = 1, TILE_RESIDUAL = 2 };

constexpr int TK = 64;                       // k-values of a stage
constexpr int ROW_BYTES = TK * 2;            // a row of a stage in LDS
constexpr int ROW_CHUNKS = ROW_BYTES / 16;   // 16-byte chunks of such a row
constexpr int ROWS_AN_INSTRUCTION = 1024 / ROW_BYTES;
constexpr int SUB_STEPS = TK / 16;           // matrix instructions' k-steps in a stage
constexpr int LDS_BYTES = 160 * 1024;
constexpr int TILE_WAVES = 8;
constexpr int TILE_THREADS = TILE_WAVES * WAVE;
constexpr int DIES = 8;

struct TileNorm {
    const float* ss_in;      // [M, pieces_in]: the rows of X lack the factor 1 / sqrt(sum / width_in + eps_in); or null
    int pieces_in;
    float eps_in;
    int width_in;
    float* resid;            // TILE_RESIDUAL: [M, N] float32, updated in place
    const float* w_out;      // [N]: the next norm's weight
    float* ss_out;           // [M, feature tiles]: each tile's share of the rows' sums of squares
};

__device__ __forceinline__ void row_chunk_into_lds(const void* from, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(from), "s"(lds_base) : "m0", "memory");
}
// s_waitcnt vmcnt(N): loads come back in order, so "all but the N youngest" is a stage's rows with the later stages'
// still on their way.  (vmcnt is six bits: the low four in bits 0..3, the high two in bits 14..15.)
template <int N> __device__ __forceinline__ void all_but_the_youngest_have_arrived() {
    static_assert(N >= 0 && N < 64, "vmcnt has six bits");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

template <int TOK, int FEAT, int WAVES_F, typename TC, int EPI>
__global__ __launch_bounds__(TILE_THREADS) void linear_tile_kernel(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                                                                   TC* __restrict__ C, int M, int N, int K, int tiles_t,
                                                                   int tiles_f, TileNorm norm) {
    constexpr int WAVES_T = TILE_WAVES / WAVES_F;
    constexpr int NF = FEAT / WAVES_F / 32, NT = TOK / WAVES_T / 32;
    constexpr int ROWS = FEAT + TOK, STAGE = ROWS * ROW_BYTES, PER_WAVE = ROWS / ROWS_AN_INSTRUCTION / TILE_WAVES;
    constexpr int RING = (LDS_BYTES - 8 * 1024) / STAGE > 6 ? 6 : (LDS_BYTES - 8 * 1024) / STAGE;      // stages in LDS
    constexpr int AHEAD = RING - 1;                                                                      // of which on their way
    static_assert(FEAT % (32 * WAVES_F) == 0 && TOK % (32 * WAVES_T) == 0 && ROWS % (ROWS_AN_INSTRUCTION * TILE_WAVES) == 0,
                  "tile and waves do not fit");
    static_assert(EPI != TILE_SWIGLU || NF % 2 == 0, "a gated tile needs gate and up features in every wave");
    static_assert(RING >= 2 && (AHEAD - 1) * PER_WAVE < 64, "the ring does not fit LDS or the load counter");
    __shared__ __attribute__((aligned(1024))) char lds[RING * STAGE];

    // which tile: blocks pid, pid + 8, .. run on one die; give each die a run of neighbouring tiles
    const int total = tiles_t * tiles_f, per_die = (total + DIES - 1) / DIES;
    const int pid = (blockIdx.x % DIES) * per_die + blockIdx.x / DIES;
    if (pid >= total) return;
    // this block's range of K, in stages, and the plane its sums go to
    const int all_stages = K / TK, per_range = (all_stages + (int)gridDim.y - 1) / (int)gridDim.y;
    const int first_stage = blockIdx.y * per_range, stages = min(per_range, all_stages - first_stage);
    if (EPI == TILE_STORE) C += (size_t)blockIdx.y * M * N;
    const int tile_t = pid % tiles_t, tile_f = pid / tiles_t;       // the token tiles of a feature tile side by side
    const int t0 = tile_t * TOK;
    const int out_feats = EPI == TILE_SWIGLU ? N / 2 : N;           // features of the result
    const int f0 = tile_f * (EPI == TILE_SWIGLU ? FEAT / 2 : FEAT);

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
            int wrow;
            if (EPI == TILE_SWIGLU) wrow = R < FEAT / 2 ? min(f0 + R, out_feats - 1) : out_feats + min(f0 + R - FEAT / 2, out_feats - 1);
            else wrow = min(f0 + R, N - 1);
            row = W + (size_t)wrow * K;
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
        int row;
        if (EPI == TILE_SWIGLU) row = (f / (NF / 2)) * (FEAT / 2) + wave_f * (FEAT / 2 / WAVES_F) + (f % (NF / 2)) * 32 + lane % 32;
        else row = wave_f * (FEAT / WAVES_F) + f * 32 + lane % 32;
        w_off[f] = row * ROW_BYTES;
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
    __syncthreads();                                           // the epilogue may use LDS: everyone is past the last stage

    // ---- epilogue.  Element v of a result tile: token lane % 32, feature 8 (v / 4) + 4 (lane / 32) + v % 4.
    int tok[NT];
    float factor[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        tok[t] = t0 + wave_t * (TOK / WAVES_T) + t * 32 + lane % 32;
        factor[t] = 1.0f;
        if (norm.ss_in) {                                      // the pieces of the row's sum of squares, in their order
            const float* p = norm.ss_in + (size_t)min(tok[t], M - 1) * norm.pieces_in;
            float sum = 0.f;
            for (int i = 0; i < norm.pieces_in; ++i) sum += p[i];
            factor[t] = 1.0f / sqrtf(sum / (float)norm.width_in + norm.eps_in);
        }
    }
    if (EPI == TILE_SWIGLU) {
#pragma unroll
        for (int f = 0; f < NF / 2; ++f)
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    const int feat = f0 + wave_f * (FEAT / 2 / WAVES_F) + f * 32 + 8 * q4 + 4 * (lane / 32);
                    float o[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float gate = acc[f][t][4 * q4 + i] * factor[t], up = acc[f + NF / 2][t][4 * q4 + i] * factor[t];
                        o[i] = gate / (1.0f + __expf(-gate)) * up;
                    }
                    if (tok[t] < M) {
                        TC* dst = C + (size_t)tok[t] * out_feats + feat;
                        if (feat + 3 < out_feats && out_feats % 4 == 0) {
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
                                if (feat + i < out_feats) dst[i] = from_float<TC>(o[i]);
                        }
                    }
                }
        return;
    }
    float sq[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) sq[t] = 0.f;
#pragma unroll
    for (int f = 0; f < NF; ++f)
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const int feat = f0 + wave_f * (FEAT / WAVES_F) + f * 32 + 8 * q4 + 4 * (lane / 32);
                float o[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) o[i] = acc[f][t][4 * q4 + i] * factor[t];
                const bool whole = feat + 3 < N && N % 4 == 0;
                if (tok[t] < M && feat < N) {
                    const size_t at = (size_t)tok[t] * N + feat;
                    if (EPI == TILE_RESIDUAL) {
                        if (whole) {
                            const float4 xo = *reinterpret_cast<const float4*>(norm.resid + at);
                            const float4 wn = *reinterpret_cast<const float4*>(norm.w_out + feat);
                            o[0] += xo.x; o[1] += xo.y; o[2] += xo.z; o[3] += xo.w;
                            *reinterpret_cast<float4*>(norm.resid + at) = make_float4(o[0], o[1], o[2], o[3]);
                            sq[t] += o[0] * o[0] + o[1] * o[1] + o[2] * o[2] + o[3] * o[3];
                            o[0] *= wn.x; o[1] *= wn.y; o[2] *= wn.z; o[3] *= wn.w;
                        } else {
#pragma unroll
                            for (int i = 0; i < 4; ++i)
                                if (feat + i < N) {
                                    o[i] += norm.resid[at + i];
                                    norm.resid[at + i] = o[i];
                                    sq[t] += o[i] * o[i];
                                    o[i] *= norm.w_out[feat + i];
                                }
                        }
                    }
                    TC* dst = C + at;
                    if (whole) {
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
    if (EPI == TILE_RESIDUAL) {
        // a token's sum of squares over this tile's features: the two halves of a wave, then the waves that share
        // the token, in a fixed order
        float* red = reinterpret_cast<float*>(lds);               // [WAVES_F][TOK]; every wave is past its last stage
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const float both = sq[t] + __shfl_xor(sq[t], 32, WAVE);
            if (lane < 32) red[wave_f * TOK + wave_t * (TOK / WAVES_T) + t * 32 + lane] = both;
        }
        __syncthreads();
        for (int i = threadIdx.x; i < TOK; i += TILE_THREADS) {
            float sum = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES_F; ++w) sum += red[w * TOK + i];
            if (t0 + i < M) norm.ss_out[(size_t)(t0 + i) * tiles_f + tile_f] = sum;
        }
    }
}

// ---- launch -----------------------------------------------------------------------------------------
constexpr int TILE_FEAT = 256;

template <int TOK, int WAVES_F, typename TC, int EPI>
static void launch_tile(hipStream_t stream, const void* x, const void* w, void* c, int M, int N, int K, int parts,
                        const TileNorm& norm) {
    const int feats_a_tile = EPI == TILE_SWIGLU ? TILE_FEAT / 2 : TILE_FEAT;
    const int out_feats = EPI == TILE_SWIGLU ? N / 2 : N;
    const int tiles_t = (M + TOK - 1) / TOK, tiles_f = (out_feats + feats_a_tile - 1) / feats_a_tile;
    const int total = tiles_t * tiles_f, blocks = (total + DIES - 1) / DIES * DIES;
    linear_tile_kernel<TOK, TILE_FEAT, WAVES_F, TC, EPI><<<dim3(blocks, parts), TILE_THREADS, 0, stream>>>(
        (const bf16_t*)x, (const bf16_t*)w, (TC*)c, M, N, K, tiles_t, tiles_f, norm);
}

// How many tokens a block takes: 256 where that still gives most compute units a block, else 128.
static int tile_tokens(int M, int out_feats, int feats_a_tile, int parts) {
    const int tiles_f = (out_feats + feats_a_tile - 1) / feats_a_tile;
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

template <typename TC, int EPI>
static void dispatch_tile(hipStream_t stream, const void* x, const void* w, void* c, int M, int N, int K, int parts,
                          const TileNorm& norm) {
    const int out_feats = EPI == TILE_SWIGLU ? N / 2 : N;
    if (tile_tokens(M, out_feats, EPI == TILE_SWIGLU ? TILE_FEAT / 2 : TILE_FEAT, parts) == 256)
        launch_tile<256, 2, TC, EPI>(stream, x, w, c, M, N, K, parts, norm);
    else
        launch_tile<128, 4, TC, EPI>(stream, x, w, c, M, N, K, parts, norm);
}

// The pieces a row's sum of squares comes in (TILE_RESIDUAL): one for each tile of 256 features.
PALM_API int palm_linear_tile_pieces(int N) { return (N + TILE_FEAT - 1) / TILE_FEAT; }

// x [M, K] bfloat16, w [N, K] bfloat16, K a multiple of 64.
//   TILE_STORE:    c [M, N] bfloat16 or float32; or, with parts > 1 (at most palm_linear_tile_parts(M, N, K)), float32
//                  planes [parts, M, N], each the sum over one range of K, for a reader that adds them in their order.
//   TILE_SWIGLU:   w is [gate rows | up rows]; c [M, N / 2] = silu(x gate^T) * (x up^T).
//   TILE_RESIDUAL: resid [M, N] float32 += x w^T; c [M, N] bfloat16 = resid * w_out (the next norm's output but for
//                  its row factor); ss_out [M, palm_linear_tile_pieces(N)] the pieces of each row's sum of squares.
// ss_in [M, pieces_in] with eps_in: the rows of x lack the factor 1 / sqrt(sum of pieces / K + eps_in), which the
// result rows get instead.
PALM_API int palm_linear_tile(hipStream_t stream, const void* x, const void* w, void* c, int c_dtype, int M, int N, int K,
                              int epilogue, int parts, const float* ss_in, int pieces_in, float eps_in, float* resid,
                              const float* w_out, float* ss_out) {
    PALM_CHECK(M >= 0 && N > 0 && K > 0, "linear_tile: M=%d N=%d K=%d", M, N, K);
    PALM_CHECK(K % TK == 0, "linear_tile: K = %d is not a multiple of %d", K, TK);
    PALM_CHECK(parts >= 1 && (parts == 1 || (epilogue == TILE_STORE && c_dtype == PALM_F32 && parts <= 4 && K / TK >= parts)),
               "linear_tile: %d planes of partial sums (they are float32, of a plain product, at most four)", parts);
    PALM_CHECK(epilogue >= TILE_STORE && epilogue <= TILE_RESIDUAL, "linear_tile: epilogue %d", epilogue);
    PALM_CHECK(epilogue != TILE_SWIGLU || N % 2 == 0, "linear_tile: a gated product needs an even N, got %d", N);
    PALM_CHECK(c_dtype == PALM_BF16 || c_dtype == PALM_F32, "linear_tile: result type %d", c_dtype);
    PALM_CHECK(((uintptr_t)x | (uintptr_t)w | (uintptr_t)c) % 16 == 0, "linear_tile: operands must be 16-byte aligned");
    PALM_CHECK(!ss_in || pieces_in > 0, "linear_tile: %d pieces of the rows' sums of squares", pieces_in);
    PALM_CHECK(epilogue != TILE_RESIDUAL || (resid && w_out && ss_out && c_dtype == PALM_BF16 && ((uintptr_t)resid | (uintptr_t)w_out) % 16 == 0),
               "linear_tile: adding to the residual stream needs the stream, the next norm's weight, room for the sums of "
               "squares and a bfloat16 result");
    PALM_CHECK((double)M * N < 2.0e9 * 4, "linear_tile: the result is beyond this kernel's index range");
    if (M == 0) return 0;
    TileNorm norm{ss_in, pieces_in, eps_in, K, resid, w_out, ss_out};
    if (epilogue == TILE_SWIGLU) {
        PALM_DTYPE_SWITCH(c_dtype, TC, dispatch_tile<TC, TILE_SWIGLU>(stream, x, w, c, M, N, K, 1, norm));
    } else if (epilogue == TILE_RESIDUAL) {
        dispatch_tile<bf16_t, TILE_RESIDUAL>(stream, x, w, c, M, N, K, 1, norm);
    } else {
        PALM_DTYPE_SWITCH(c_dtype, TC, dispatch_tile<TC, TILE_STORE>(stream, x, w, c, M, N, K, parts, norm));
    }
    PALM_LAUNCHED();
    return 0;
}
