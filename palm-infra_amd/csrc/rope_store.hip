// Per-head RMSNorm of q and k, rotation of both, and the write of k and v into the paged cache, in one
// pass over the projection's output.
//
// The reference does this as separate graph nodes: reshape/permute copies, rms_norm over head_dim rows
// with one weight for all heads, rope with per-position cos/sin rows, and the append inside SDPA
// (models/qwen3.py:310-334; kernels/rope.cpp:38-48; engine/cuda_attention.cu:8-113).  Angles are
// position * inv_freq in 32-bit with full-range sin/cos (engine/input_prep.cpp:17-30).  As in the
// reference's graph (models/qwen3.py:226-227) the rotation comes in as cos/sin rows for the step's
// tokens, made once per step by the part that owns the position encoding.
//
// Layouts: qkv [n_tokens, (nh + 2 nkv) * hd] as the projection writes it (q heads, k heads, v heads);
// q_out [n_tokens, nh * hd]; key cache [pages, nkv, PAGE_TOKENS, hd]; value cache transposed,
// [pages, nkv, hd, PAGE_TOKENS] (the attention kernels sum over keys, which must be contiguous for the
// matrix cores); page of position p of a slot is block_table[slot * max_pages + p / PAGE_TOKENS].
#include "common.h"

#include <type_traits>

constexpr int MAX_HEAD_DIM = 512;
// From here on the kernels for many tokens run, where they serve the head size and q/k/v come whole, not as
// planes.  Measured at 32 heads of 128 over 8 kv heads: 256 tokens 8.6 to 10 us with one wave a head against 10 to
// 17 us, 512 tokens 14.5 to 18 against 11 to 18 (the slower figures: every token in a sequence of its own).
constexpr int FAST_MIN_TOKENS = 384;

// One wave per (token, head).  pairing 0: pairs (i, i + rot/2); pairing 1: pairs (2i, 2i + 1).
// qkv may come as `planes` planes of partial sums (a projection that cut its K into ranges), plane_stride
// elements apart; they are added in their order.
template <typename TIN, typename T>
__global__ __launch_bounds__(WAVE) void qk_norm_rope_store_kernel(
    const TIN* __restrict__ qkv, int planes, size_t plane_stride,
    T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ tok_slot,
    const int* __restrict__ positions, const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w,
    float eps, const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rotary_dim, int pairing,
    int nh, int nkv, int hd,
    int write_cache, float q_scale) {
    __shared__ float vals[MAX_HEAD_DIM];
    const int t = blockIdx.x;
    const int head = blockIdx.y;                 // 0..nh-1: q, then nkv k heads, then nkv v heads
    const int lane = threadIdx.x;
    const int kind = head < nh ? 0 : (head < nh + nkv ? 1 : 2);
    if (kind != 0 && !write_cache) return;
    const TIN* src = qkv + ((size_t)t * (nh + 2 * nkv) + head) * hd;
    // What does not depend on the row is asked for first (the position, its page, the first rotation pair's cos and
    // sin, the norm weight): the kernel's time is the round trips to memory that follow each other.
    const int pos = positions[t];
    const bool rotate = kind != 2 && cos_t && rotary_dim > 0;
    const int half = rotary_dim / 2;
    float c0 = 1.f, s0 = 0.f;
    if (rotate && lane < half) {
        c0 = cos_t[(size_t)t * half + lane];
        s0 = sin_t[(size_t)t * half + lane];
    }
    int page = 0;
    if (kind != 0) page = block_table[(size_t)tok_slot[t] * max_pages + pos / PAGE_TOKENS];
    const float* norm_w = kind == 0 ? q_norm_w : (kind == 1 ? k_norm_w : nullptr);
    const float w0 = norm_w && lane < hd ? norm_w[lane] : 1.f;

    float ss = 0.f;
    for (int d = lane; d < hd; d += WAVE) {
        float v = to_float(src[d]);
        for (int p = 1; p < planes; ++p) v += to_float(src[p * plane_stride + d]);
        vals[d] = v;
        ss += v * v;
    }
    if (norm_w) {
        ss = wave_sum(ss);
        const float inv = 1.0f / sqrtf(ss / (float)hd + eps);
        for (int d = lane; d < hd; d += WAVE) vals[d] = vals[d] * inv * (d == lane ? w0 : norm_w[d]);
    }
    __syncthreads();

    if (rotate) {
        for (int i = lane; i < half; i += WAVE) {
            const int a = pairing == 0 ? i : 2 * i;
            const int b = pairing == 0 ? i + half : 2 * i + 1;
            const float c = i == lane ? c0 : cos_t[(size_t)t * half + i], s = i == lane ? s0 : sin_t[(size_t)t * half + i];
            const float x0 = vals[a], x1 = vals[b];
            vals[a] = x0 * c - x1 * s;
            vals[b] = x0 * s + x1 * c;
        }
        __syncthreads();
    }

    if (kind == 2) {
        const int g = head - nh - nkv;
        T* dst = v_cache + ((size_t)page * nkv + g) * hd * PAGE_TOKENS + pos % PAGE_TOKENS;
        for (int d = lane; d < hd; d += WAVE) dst[(size_t)d * PAGE_TOKENS] = from_float<T>(vals[d]);
        return;
    }
    T* dst;
    float scale = 1.0f;
    if (kind == 0) {
        dst = q_out + ((size_t)t * nh + head) * hd;
        scale = q_scale;                         // what the attention kernel wants folded into the queries before they are rounded
    } else {
        const int g = head - nh;
        dst = k_cache + (((size_t)page * nkv + g) * PAGE_TOKENS + pos % PAGE_TOKENS) * hd;
    }
    for (int d = lane; d < hd; d += WAVE) dst[d] = from_float<T>(vals[d] * scale);
}

// ---- the same for many tokens (prompts) -------------------------------------------------------------
// With thousands of tokens the kernel above is bound by its own bookkeeping: a block for every (token,
// head), values through LDS, and for v a store of two bytes every 128.  Here
//   q and k: a head is held by L lanes with E = hd / L elements each, 64 / L heads a wave: E as large as it can be
//            (at most 8) with L a power of two, because a wave's instruction costs the same for two elements a
//            lane as for eight (at head size 128: E = 8, L = 16, four heads a wave).  The rotation partner of
//            element d, d +- hd/2, is then element e of lane l ^ (L/2), one shuffle away, and the row's sum of
//            squares is a shuffle tree over L lanes: no LDS, no barrier.
//   v:       a block takes 64 consecutive tokens of one kv head, lays them into LDS and writes them with one
//            lane a token, so that tokens side by side in a page are written side by side.
// Served (rope_fast_serves): E <= 8, and a rotation that keeps a pair inside a lane or with the partner lane:
// half-split over the whole head, interleaved with an even E, or none.
constexpr int FAST_MAX_E = 8;

// lanes a head: hd / E for the largest E <= 8 that leaves a power of two of at least 2 and at most 64 lanes; 0 if none
static int fast_lanes(int hd) {
    for (int E = FAST_MAX_E; E >= 1; --E) {
        if (hd % E) continue;
        const int L = hd / E;
        if (L >= 2 && L <= 64 && (L & (L - 1)) == 0) return L;
    }
    return 0;
}
static bool rope_fast_serves(int hd, int rotary_dim, int pairing, bool has_rotation) {
    const int L = fast_lanes(hd);
    if (L == 0) return false;
    const int E = hd / L;
    if (!has_rotation || rotary_dim == 0) return true;
    return pairing == 0 ? rotary_dim == hd : E % 2 == 0;
}

// E consecutive elements, read or written with the widest access their number allows
template <int E> __device__ inline void read_elems(const float* p, float (&x)[E]) {
    if constexpr (E % 4 == 0) {
#pragma unroll
        for (int i = 0; i < E; i += 4) {
            const float4 v = *reinterpret_cast<const float4*>(p + i);
            x[i] = v.x; x[i + 1] = v.y; x[i + 2] = v.z; x[i + 3] = v.w;
        }
    } else if constexpr (E % 2 == 0) {
#pragma unroll
        for (int i = 0; i < E; i += 2) {
            const float2 v = *reinterpret_cast<const float2*>(p + i);
            x[i] = v.x; x[i + 1] = v.y;
        }
    } else {
#pragma unroll
        for (int i = 0; i < E; ++i) x[i] = p[i];
    }
}
template <int E> __device__ inline void read_elems(const bf16_t* p, float (&x)[E]) {
    if constexpr (E % 2 == 0) {
#pragma unroll
        for (int i = 0; i < E; i += 2) {
            const uint32_t u = *reinterpret_cast<const uint32_t*>(p + i);
            x[i] = __uint_as_float(u << 16);
            x[i + 1] = __uint_as_float(u & 0xffff0000u);
        }
    } else {
#pragma unroll
        for (int i = 0; i < E; ++i) x[i] = to_float(p[i]);
    }
}
template <int E> __device__ inline void write_elems(float* p, const float (&x)[E]) {
#pragma unroll
    for (int i = 0; i < E; ++i) p[i] = x[i];
}
template <int E> __device__ inline void write_elems(bf16_t* p, const float (&x)[E]) {
    if constexpr (E % 2 == 0) {
#pragma unroll
        for (int i = 0; i < E; i += 2)
            *reinterpret_cast<uint32_t*>(p + i) = (uint32_t)f32_to_bf16(x[i]).bits | ((uint32_t)f32_to_bf16(x[i + 1]).bits << 16);
    } else {
#pragma unroll
        for (int i = 0; i < E; ++i) p[i] = f32_to_bf16(x[i]);
    }
}

// One block a token.  What does not depend on the head (norm weights, the token's cos/sin, its page) is read
// once; then every wave takes heads four at a time, all four reads on their way before the first is used:
// the kernel's time is the latency of its reads, so they must not wait for each other.
constexpr int FAST_HEADS_AT_ONCE = 4;

template <typename TIN, typename T, int E>
__global__ __launch_bounds__(4 * WAVE) void qk_norm_rope_fast_kernel(
    const TIN* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ k_cache,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ tok_slot,
    const int* __restrict__ positions, const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w,
    float eps, const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rotary_dim, int pairing,
    int nh, int nkv, int hd, int L, int write_cache, float q_scale) {
    constexpr int U = FAST_HEADS_AT_ONCE;
    const int t = blockIdx.x;
    const int per_wave = WAVE / L;
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    const int l = lane % L, sub = lane / L;                   // this lane's place in its head, its head's place in the wave
    const int n_heads = write_cache ? nh + nkv : nh;          // q heads, then k heads
    const bool rotate = cos_t && rotary_dim > 0;
    const int half = rotary_dim / 2;
    const bool low = l < L / 2;

    float wq[E], wk[E], c[E], sn[E];
    if (q_norm_w) {                                           // q and k norms come together
        read_elems<E>(q_norm_w + l * E, wq);
        read_elems<E>(k_norm_w + l * E, wk);
    }
    if (rotate && pairing == 0) {                             // (i, i + hd/2): the partner is element e of lane l ^ (L/2)
        const int i0 = (low ? l : l - L / 2) * E;
        read_elems<E>(cos_t + (size_t)t * half + i0, c);
        read_elems<E>(sin_t + (size_t)t * half + i0, sn);
    } else if (rotate) {                                      // (2i, 2i + 1), both in this lane: E is even
#pragma unroll
        for (int e = 0; e < E; e += 2) {
            const int d = l * E + e, i = d < rotary_dim ? d / 2 : 0;
            c[e] = cos_t[(size_t)t * half + i];
            sn[e] = sin_t[(size_t)t * half + i];
        }
    }
    size_t k_row = 0;
    if (write_cache) {
        const int pos = positions[t];
        const int page = block_table[(size_t)tok_slot[t] * max_pages + pos / PAGE_TOKENS];
        k_row = ((size_t)page * nkv * PAGE_TOKENS + pos % PAGE_TOKENS) * hd;
    }
    const TIN* token = qkv + (size_t)t * (nh + 2 * nkv) * hd + l * E;

    for (int base = 0; base < n_heads; base += U * 4 * per_wave) {
        float x[U][E];
        int head[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            head[u] = base + (u * 4 + wave) * per_wave + sub;
            read_elems<E>(token + (size_t)min(head[u], n_heads - 1) * hd, x[u]);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (base + (u * 4 + wave) * per_wave >= n_heads) continue;       // none of the wave's heads of this turn exists
            const bool is_k = head[u] >= nh;
            if (q_norm_w) {
                float ss = 0.f;
#pragma unroll
                for (int e = 0; e < E; ++e) ss += x[u][e] * x[u][e];
                if (L == 64) {
#pragma unroll
                    for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, WAVE);
                } else {
                    for (int off = L / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, WAVE);
                }
                const float inv = 1.0f / sqrtf(ss / (float)hd + eps);
#pragma unroll
                for (int e = 0; e < E; ++e) x[u][e] = x[u][e] * inv * (is_k ? wk[e] : wq[e]);
            }
            if (rotate && pairing == 0) {
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    const float other = L == 64 ? __shfl_xor(x[u][e], 32, WAVE) : __shfl_xor(x[u][e], L / 2, WAVE);
                    x[u][e] = low ? x[u][e] * c[e] - other * sn[e] : other * sn[e] + x[u][e] * c[e];
                }
            } else if (rotate) {
                if constexpr (E % 2 == 0) {
#pragma unroll
                    for (int e = 0; e < E; e += 2) {
                        const bool turn = l * E + e < rotary_dim;
                        const float x0 = x[u][e], x1 = x[u][e + 1];
                        x[u][e] = turn ? x0 * c[e] - x1 * sn[e] : x0;
                        x[u][e + 1] = turn ? x0 * sn[e] + x1 * c[e] : x1;
                    }
                }
            }
            if (!is_k) {
#pragma unroll
                for (int e = 0; e < E; ++e) x[u][e] *= q_scale;
            }
            if (head[u] < n_heads) {
                T* dst = is_k ? k_cache + k_row + (size_t)(head[u] - nh) * PAGE_TOKENS * hd : q_out + ((size_t)t * nh + head[u]) * hd;
                write_elems<E>(dst + l * E, x[u]);
            }
        }
    }
}

// v of 64 consecutive tokens of one kv head into the transposed pages
template <typename TIN, typename T>
__global__ __launch_bounds__(4 * WAVE) void v_store_tile_kernel(
    const TIN* __restrict__ qkv, T* __restrict__ v_cache,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ tok_slot,
    const int* __restrict__ positions, int n_tokens, int nh, int nkv, int hd) {
    __shared__ float tile[PAGE_TOKENS][33];                  // 32 elements of 64 tokens at a time
    const int t0 = blockIdx.x * PAGE_TOKENS, g = blockIdx.y;
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    // the lane's own token, for the writes
    const int t_mine = min(t0 + lane, n_tokens - 1);
    const int pos = positions[t_mine];
    const int page = block_table[(size_t)tok_slot[t_mine] * max_pages + pos / PAGE_TOKENS];
    T* dst = v_cache + ((size_t)page * nkv + g) * hd * PAGE_TOKENS + pos % PAGE_TOKENS;
    if constexpr (std::is_same<TIN, bf16_t>::value && std::is_same<T, bf16_t>::value) {
        if (hd % 8 == 0) {
            // bfloat16 straight through: 128 elements of the 64 tokens at a time, read 16 bytes a thread, kept in LDS
            // as pairs (rows of 65 words: a lane a token then reads without a bank conflict), written two rows a read
            __shared__ uint32_t pairs[PAGE_TOKENS][65];
            for (int d0 = 0; d0 < hd; d0 += 128) {
                const int chunks = min(128, hd - d0) / 8;         // 16-byte chunks of a token's row in this pass
                uint4 got[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int i = k * 4 * WAVE + threadIdx.x, tt = i / 16, ch = i % 16;
                    const bool ok = ch < chunks && t0 + tt < n_tokens;
                    const bf16_t* src = qkv + ((size_t)min(t0 + tt, n_tokens - 1) * (nh + 2 * nkv) + nh + nkv + g) * hd + d0 + (ok ? ch : 0) * 8;
                    got[k] = *reinterpret_cast<const uint4*>(src);
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int i = k * 4 * WAVE + threadIdx.x, tt = i / 16, ch = i % 16;
                    pairs[tt][ch * 4 + 0] = got[k].x; pairs[tt][ch * 4 + 1] = got[k].y;
                    pairs[tt][ch * 4 + 2] = got[k].z; pairs[tt][ch * 4 + 3] = got[k].w;
                }
                __syncthreads();
                if (t0 + lane < n_tokens) {
                    for (int w = wave; w < chunks * 4; w += 4) {
                        const uint32_t two = pairs[lane][w];
                        bf16_t lo, hi;
                        lo.bits = (uint16_t)(two & 0xffffu);
                        hi.bits = (uint16_t)(two >> 16);
                        dst[(size_t)(d0 + 2 * w) * PAGE_TOKENS] = lo;
                        dst[(size_t)(d0 + 2 * w + 1) * PAGE_TOKENS] = hi;
                    }
                }
                __syncthreads();
            }
            return;
        }
    }
    for (int d0 = 0; d0 < hd; d0 += 32) {
        // read: 8 tokens at a time for each wave, 32 elements side by side (two passes fill the 16 of a wave)
        for (int i = threadIdx.x; i < PAGE_TOKENS * 32; i += 4 * WAVE) {
            const int tt = i / 32, d = d0 + i % 32;
            float v = 0.f;
            if (t0 + tt < n_tokens && d < hd) {
                const TIN* src = qkv + ((size_t)(t0 + tt) * (nh + 2 * nkv) + nh + nkv + g) * hd + d;
                v = to_float(*src);
            }
            tile[tt][i % 32] = v;
        }
        __syncthreads();
        for (int dd = wave; dd < 32; dd += 4) {
            const int d = d0 + dd;
            if (d < hd && t0 + lane < n_tokens) dst[(size_t)d * PAGE_TOKENS] = from_float<T>(tile[lane][dd]);
        }
        __syncthreads();
    }
}

// dtype: the element type of q_out and of the cache, and of qkv if planes == 1; with planes > 1 qkv is
// [planes, n_tokens, (nh + 2 nkv) * hd] float32.  q_scale: a factor on the queries (not the keys), applied in 32-bit
// before they are rounded: 1, or what the attention kernel that reads them wants folded in.
PALM_API int palm_qk_norm_rope_store(hipStream_t stream, const void* qkv, int dtype, int planes, void* q_out, void* k_cache,
                                     void* v_cache, const int* block_table, int max_pages, const int* tok_slot,
                                     const int* positions, const float* q_norm_w, const float* k_norm_w, float eps,
                                     const float* cos_t, const float* sin_t, int rotary_dim, int pairing,
                                     int n_tokens, int nh, int nkv, int hd, int write_cache, float q_scale) {
    PALM_CHECK(n_tokens >= 0 && nh > 0 && nkv > 0 && hd > 0, "qk_norm_rope_store: tokens=%d heads=%d kv=%d hd=%d",
               n_tokens, nh, nkv, hd);
    PALM_CHECK(hd <= MAX_HEAD_DIM, "qk_norm_rope_store: head_dim %d exceeds %d", hd, MAX_HEAD_DIM);
    PALM_CHECK(rotary_dim >= 0 && rotary_dim <= hd && rotary_dim % 2 == 0,
               "qk_norm_rope_store: rotary_dim %d must be even and at most head_dim %d", rotary_dim, hd);
    PALM_CHECK(pairing == 0 || pairing == 1, "qk_norm_rope_store: pairing %d is neither half-split (0) nor interleaved (1)", pairing);
    PALM_CHECK((cos_t == nullptr) == (sin_t == nullptr), "qk_norm_rope_store: cos and sin tables come together");
    PALM_CHECK(!write_cache || (k_cache && v_cache && block_table && tok_slot && max_pages > 0),
               "qk_norm_rope_store: a cache write needs the cache, the page table and the slots");
    PALM_CHECK(planes >= 1, "qk_norm_rope_store: %d planes", planes);
    if (n_tokens == 0) return 0;
    dim3 grid(n_tokens, nh + 2 * nkv);
    PALM_CHECK(grid.y <= 65535, "qk_norm_rope_store: %d heads are more than one launch takes", (int)grid.y);
    const size_t plane_stride = (size_t)n_tokens * (nh + 2 * nkv) * hd;
    if (planes == 1 && n_tokens >= FAST_MIN_TOKENS && rope_fast_serves(hd, rotary_dim, pairing, cos_t != nullptr)) {
        const int L = fast_lanes(hd);
        const dim3 qk_grid(n_tokens);
        const dim3 v_grid((n_tokens + PAGE_TOKENS - 1) / PAGE_TOKENS, nkv);
        PALM_CHECK(v_grid.y <= 65535, "qk_norm_rope_store: %d kv heads are more than one launch takes", nkv);
#define PALM_ROPE_FAST_E(TIN, T, EE) case EE: \
        qk_norm_rope_fast_kernel<TIN, T, EE><<<qk_grid, 4 * WAVE, 0, stream>>>( \
            (const TIN*)qkv, (T*)q_out, (T*)k_cache, block_table, max_pages, tok_slot, positions, \
            q_norm_w, k_norm_w, eps, cos_t, sin_t, rotary_dim, pairing, nh, nkv, hd, L, write_cache, q_scale); break;
#define PALM_ROPE_FAST(TIN, T) do { \
        switch (hd / L) { \
            PALM_ROPE_FAST_E(TIN, T, 1) PALM_ROPE_FAST_E(TIN, T, 2) PALM_ROPE_FAST_E(TIN, T, 3) PALM_ROPE_FAST_E(TIN, T, 4) \
            PALM_ROPE_FAST_E(TIN, T, 5) PALM_ROPE_FAST_E(TIN, T, 6) PALM_ROPE_FAST_E(TIN, T, 7) PALM_ROPE_FAST_E(TIN, T, 8) \
        } \
        if (write_cache) v_store_tile_kernel<TIN, T><<<v_grid, 4 * WAVE, 0, stream>>>( \
            (const TIN*)qkv, (T*)v_cache, block_table, max_pages, tok_slot, positions, n_tokens, nh, nkv, hd); \
    } while (0)
        PALM_DTYPE_SWITCH(dtype, T, PALM_ROPE_FAST(T, T));
#undef PALM_ROPE_FAST_E
#undef PALM_ROPE_FAST
        PALM_LAUNCHED();
        return 0;
    }
    if (planes > 1) {
        PALM_DTYPE_SWITCH(dtype, T,
            (qk_norm_rope_store_kernel<float, T><<<grid, WAVE, 0, stream>>>(
                (const float*)qkv, planes, plane_stride, (T*)q_out, (T*)k_cache, (T*)v_cache, block_table, max_pages,
                tok_slot, positions, q_norm_w, k_norm_w, eps, cos_t, sin_t, rotary_dim, pairing, nh, nkv, hd, write_cache, q_scale)));
    } else {
        PALM_DTYPE_SWITCH(dtype, T,
            (qk_norm_rope_store_kernel<T, T><<<grid, WAVE, 0, stream>>>(
                (const T*)qkv, 1, plane_stride, (T*)q_out, (T*)k_cache, (T*)v_cache, block_table, max_pages,
                tok_slot, positions, q_norm_w, k_norm_w, eps, cos_t, sin_t, rotary_dim, pairing, nh, nkv, hd, write_cache, q_scale)));
    }
    PALM_LAUNCHED();
    return 0;
}

// cos/sin rows [n_tokens, half] for the step's positions: angle = position * inv_freq[i], in 32-bit,
// with the full-range sin and cos (engine/input_prep.cpp:17-30).
__global__ void rope_table_kernel(const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                  float* __restrict__ cos_t, float* __restrict__ sin_t, int n_tokens, int half) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_tokens * half) return;
    const float ang = (float)positions[i / half] * inv_freq[i % half];
    float s, c;
    sincosf(ang, &s, &c);
    cos_t[i] = c;
    sin_t[i] = s;
}

PALM_API int palm_rope_table(hipStream_t stream, const int* positions, const float* inv_freq, float* cos_t,
                             float* sin_t, int n_tokens, int half) {
    PALM_CHECK(n_tokens >= 0 && half > 0, "rope_table: tokens=%d half=%d", n_tokens, half);
    if (n_tokens == 0) return 0;
    const long long total = (long long)n_tokens * half;
    PALM_CHECK(total < (1ll << 31), "rope_table: %lld entries are more than one launch takes", total);
    rope_table_kernel<<<(int)((total + 255) / 256), 256, 0, stream>>>(positions, inv_freq, cos_t, sin_t, n_tokens, half);
    PALM_LAUNCHED();
    return 0;
}
