// Causal grouped-query attention over the paged cache, for prompts and for single tokens, any head
// size, all arithmetic in 32-bit with full-precision exp.  This is the exact path (the float32 mode)
// and the fallback for head sizes that the matrix-core kernels do not take.
//
// Semantics (models/qwen3.py:336-341; kernels/attention.cpp:937-962; engine/input_prep.cpp:8-15):
// head h reads kv head h / (nh / nkv); s_j = scale * q . k_j for the keys j <= p of the query's own
// sequence (and j > p - window if there is a window); softmax with the running maximum subtracted;
// o = sum_j p_j v_j.  The keys of the step's own tokens are already in the cache when this runs.
// K is [pages, nkv, 64, hd]; V is kept transposed, [pages, nkv, hd, 64].
//
// One block of four waves per (query, head).  A wave takes every fourth page of the key range; inside
// a page each lane scores one key, the wave keeps a running (max, sum, output) and the four partial
// results are merged at the end.
#include "common.h"

constexpr int ATT_WAVES = 4;
constexpr int ATT_MAX_HD = 512;
constexpr int ATT_ACC = ATT_MAX_HD / WAVE;

template <typename T>
__global__ __launch_bounds__(ATT_WAVES * WAVE) void attention_simple_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_start, const int* __restrict__ seq_new, const int* __restrict__ cu_new,
    int nh, int nkv, int hd, float scale, int window, T* __restrict__ out) {
    __shared__ float q_s[ATT_MAX_HD];
    __shared__ float m_s[ATT_WAVES], l_s[ATT_WAVES];
    __shared__ float acc_s[ATT_WAVES][ATT_MAX_HD];

    const int qi = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    if (qi >= seq_new[b]) return;
    const int t = cu_new[b] + qi;
    const int pos = seq_start[b] + qi;
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int g = h / (nh / nkv);
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    const int* pages = block_table + (size_t)seq_slot[b] * max_pages;

    const T* qp = q + ((size_t)t * nh + h) * hd;
    for (int d = threadIdx.x; d < hd; d += blockDim.x) q_s[d] = to_float(qp[d]);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[ATT_ACC];
#pragma unroll
    for (int i = 0; i < ATT_ACC; ++i) acc[i] = 0.f;

    for (int pg = lo / PAGE_TOKENS + wave; pg <= pos / PAGE_TOKENS; pg += ATT_WAVES) {
        const int page = pages[pg];
        const T* kp = k_cache + ((size_t)page * nkv + g) * PAGE_TOKENS * hd;
        const T* vp = v_cache + ((size_t)page * nkv + g) * PAGE_TOKENS * hd;
        const int j = pg * PAGE_TOKENS + lane;
        float s = -INFINITY;
        if (j >= lo && j <= pos) {
            const T* kr = kp + (size_t)lane * hd;
            float dot = 0.f;
            for (int d = 0; d < hd; ++d) dot = fmaf(q_s[d], to_float(kr[d]), dot);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float alpha = expf(m - m_new);        // m = -inf at the first page: exp(-inf) = 0
        const float p = expf(s - m_new);            // an invisible key: exp(-inf) = 0
        l = l * alpha + wave_sum(p);
        m = m_new;
#pragma unroll
        for (int i = 0; i < ATT_ACC; ++i) acc[i] *= alpha;
        const int j_first = max(lo, pg * PAGE_TOKENS) - pg * PAGE_TOKENS;
        const int j_last = min(pos, pg * PAGE_TOKENS + PAGE_TOKENS - 1) - pg * PAGE_TOKENS;
        for (int jj = j_first; jj <= j_last; ++jj) {
            const float pj = __shfl(p, jj, WAVE);   // jj is the same in every lane
#pragma unroll
            for (int i = 0; i < ATT_ACC; ++i) {
                const int d = lane + i * WAVE;
                if (d < hd) acc[i] = fmaf(pj, to_float(vp[(size_t)d * PAGE_TOKENS + jj]), acc[i]);
            }
        }
    }

    if (lane == 0) { m_s[wave] = m; l_s[wave] = l; }
#pragma unroll
    for (int i = 0; i < ATT_ACC; ++i) {
        const int d = lane + i * WAVE;
        if (d < hd) acc_s[wave][d] = acc[i];
    }
    __syncthreads();
    float m_all = -INFINITY;
    for (int w = 0; w < ATT_WAVES; ++w) m_all = fmaxf(m_all, m_s[w]);
    float l_all = 0.f;
    for (int w = 0; w < ATT_WAVES; ++w) l_all += l_s[w] * expf(m_s[w] - m_all);
    T* op = out + ((size_t)t * nh + h) * hd;
    for (int d = threadIdx.x; d < hd; d += blockDim.x) {
        float o = 0.f;
        for (int w = 0; w < ATT_WAVES; ++w) o += acc_s[w][d] * expf(m_s[w] - m_all);
        op[d] = from_float<T>(o / l_all);
    }
}

PALM_API int palm_attention_simple(hipStream_t stream, const void* q, int dtype, const void* k_cache,
                                   const void* v_cache, const int* block_table, int max_pages, const int* seq_slot,
                                   const int* seq_start, const int* seq_new, const int* cu_new, int n_seqs,
                                   int max_new, int nh, int nkv, int hd, float scale, int window, void* out) {
    PALM_CHECK(n_seqs >= 0 && max_new >= 0 && nh > 0 && nkv > 0 && hd > 0,
               "attention: seqs=%d max_new=%d heads=%d kv=%d hd=%d", n_seqs, max_new, nh, nkv, hd);
    PALM_CHECK(nh % nkv == 0, "attention: %d heads are not a multiple of %d kv heads", nh, nkv);
    PALM_CHECK(hd <= ATT_MAX_HD, "attention: head_dim %d exceeds %d", hd, ATT_MAX_HD);
    PALM_CHECK(window >= 0, "attention: window %d", window);
    PALM_CHECK(max_pages > 0, "attention: max_pages %d", max_pages);
    if (n_seqs == 0 || max_new == 0) return 0;
    PALM_CHECK(nh <= 65535 && n_seqs <= 65535, "attention: %d heads / %d sequences are more than one launch takes", nh, n_seqs);
    dim3 grid(max_new, nh, n_seqs);
    PALM_DTYPE_SWITCH(dtype, T,
        attention_simple_kernel<T><<<grid, ATT_WAVES * WAVE, 0, stream>>>(
            (const T*)q, (const T*)k_cache, (const T*)v_cache, block_table, max_pages, seq_slot, seq_start, seq_new,
            cu_new, nh, nkv, hd, scale, window, (T*)out));
    PALM_LAUNCHED();
    return 0;
}
