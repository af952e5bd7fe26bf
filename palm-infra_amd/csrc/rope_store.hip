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

constexpr int MAX_HEAD_DIM = 512;

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
    int write_cache) {
    __shared__ float vals[MAX_HEAD_DIM];
    const int t = blockIdx.x;
    const int head = blockIdx.y;                 // 0..nh-1: q, then nkv k heads, then nkv v heads
    const int lane = threadIdx.x;
    const int kind = head < nh ? 0 : (head < nh + nkv ? 1 : 2);
    if (kind != 0 && !write_cache) return;
    const TIN* src = qkv + ((size_t)t * (nh + 2 * nkv) + head) * hd;

    float ss = 0.f;
    for (int d = lane; d < hd; d += WAVE) {
        float v = to_float(src[d]);
        for (int p = 1; p < planes; ++p) v += to_float(src[p * plane_stride + d]);
        vals[d] = v;
        ss += v * v;
    }
    const float* norm_w = kind == 0 ? q_norm_w : (kind == 1 ? k_norm_w : nullptr);
    if (norm_w) {
        ss = wave_sum(ss);
        const float inv = 1.0f / sqrtf(ss / (float)hd + eps);
        for (int d = lane; d < hd; d += WAVE) vals[d] = vals[d] * inv * norm_w[d];
    }
    __syncthreads();

    const int pos = positions[t];
    if (kind != 2 && cos_t && rotary_dim > 0) {
        const int half = rotary_dim / 2;
        for (int i = lane; i < half; i += WAVE) {
            const int a = pairing == 0 ? i : 2 * i;
            const int b = pairing == 0 ? i + half : 2 * i + 1;
            const float c = cos_t[(size_t)t * half + i], s = sin_t[(size_t)t * half + i];
            const float x0 = vals[a], x1 = vals[b];
            vals[a] = x0 * c - x1 * s;
            vals[b] = x0 * s + x1 * c;
        }
        __syncthreads();
    }

    if (kind == 2) {
        const int g = head - nh - nkv;
        const int page = block_table[(size_t)tok_slot[t] * max_pages + pos / PAGE_TOKENS];
        T* dst = v_cache + ((size_t)page * nkv + g) * hd * PAGE_TOKENS + pos % PAGE_TOKENS;
        for (int d = lane; d < hd; d += WAVE) dst[(size_t)d * PAGE_TOKENS] = from_float<T>(vals[d]);
        return;
    }
    T* dst;
    if (kind == 0) {
        dst = q_out + ((size_t)t * nh + head) * hd;
    } else {
        const int g = head - nh;
        const int page = block_table[(size_t)tok_slot[t] * max_pages + pos / PAGE_TOKENS];
        dst = k_cache + (((size_t)page * nkv + g) * PAGE_TOKENS + pos % PAGE_TOKENS) * hd;
    }
    for (int d = lane; d < hd; d += WAVE) dst[d] = from_float<T>(vals[d]);
}

// dtype: the element type of q_out and of the cache, and of qkv if planes == 1; with planes > 1 qkv is
// [planes, n_tokens, (nh + 2 nkv) * hd] float32.
PALM_API int palm_qk_norm_rope_store(hipStream_t stream, const void* qkv, int dtype, int planes, void* q_out, void* k_cache,
                                     void* v_cache, const int* block_table, int max_pages, const int* tok_slot,
                                     const int* positions, const float* q_norm_w, const float* k_norm_w, float eps,
                                     const float* cos_t, const float* sin_t, int rotary_dim, int pairing,
                                     int n_tokens, int nh, int nkv, int hd, int write_cache) {
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
    if (planes > 1) {
        PALM_DTYPE_SWITCH(dtype, T,
            (qk_norm_rope_store_kernel<float, T><<<grid, WAVE, 0, stream>>>(
                (const float*)qkv, planes, plane_stride, (T*)q_out, (T*)k_cache, (T*)v_cache, block_table, max_pages,
                tok_slot, positions, q_norm_w, k_norm_w, eps, cos_t, sin_t, rotary_dim, pairing, nh, nkv, hd, write_cache)));
    } else {
        PALM_DTYPE_SWITCH(dtype, T,
            (qk_norm_rope_store_kernel<T, T><<<grid, WAVE, 0, stream>>>(
                (const T*)qkv, 1, plane_stride, (T*)q_out, (T*)k_cache, (T*)v_cache, block_table, max_pages,
                tok_slot, positions, q_norm_w, k_norm_w, eps, cos_t, sin_t, rotary_dim, pairing, nh, nkv, hd, write_cache)));
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
