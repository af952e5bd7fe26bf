// Choosing the next token from a row of logits, on the device: greedy, temperature, top-k, top-p,
// min-p and the penalties of the reference's sampler (engine/sampler.cpp).
//
//   greedy      temperature <= 0 or top_k == 1: the first maximum (engine/sampler.cpp:72-77, 171-172)
//   candidates  the k largest logits, ties to the lower id (engine/sampler.cpp:93-119), sorted by
//               (logit descending, id ascending); w = exp((l - l_max) / T) (:121-124)
//   min_p       keep w >= min_p * w_best (:127-133)
//   top_p       keep the shortest sorted prefix whose mass reaches top_p * sum (:143-154)
//   draw        the first candidate whose cumulative weight reaches u * sum (:180-187)
//   penalties   l > 0 ? l / r : l * r, l -= presence, l -= frequency * count (:335-340)
//
// The uniform number u of each row comes from the caller (a counter-based generator keyed by the
// request, so a row's draw does not depend on its batch companions).  Without top_k the candidates are
// not sorted: the kept set is found by a threshold on the logit and the draw walks it in index order,
// which gives the same distribution.
#include "common.h"

constexpr int SAMPLE_THREADS = 1024;
constexpr int TOPK_MAX = 1024;

// Monotone map from float to unsigned: a larger float gives a larger key.
__device__ inline uint32_t ordered_key(float f) {
    uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct BestPair { float v; int i; };
__device__ inline BestPair better(BestPair a, BestPair b) {
    // the larger value; on equal values the lower index
    if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
    return a;
}

// argmax of one row by the whole block; every thread returns the result
__device__ BestPair block_argmax(const float* __restrict__ row, int V, BestPair* scratch) {
    BestPair best{-INFINITY, 0x7fffffff};
    // a thread's indices rise, so a tie keeps the lower one: the elements before the first 16-byte border, then
    // the body four at a time (four reads in flight), then the rest
    const int head = min(V, (int)(((16 - ((uintptr_t)row & 15)) & 15) / 4));
    const int n4 = (V - head) / 4;
    for (int i = threadIdx.x; i < head; i += blockDim.x) {
        const float v = row[i];
        if (v > best.v) { best.v = v; best.i = i; }
    }
    const float4* body = reinterpret_cast<const float4*>(row + head);
    for (int i0 = threadIdx.x; i0 < n4; i0 += 4 * blockDim.x) {
        float4 q[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) q[u] = body[min(i0 + u * (int)blockDim.x, n4 - 1)];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i4 = i0 + u * (int)blockDim.x;
            if (i4 >= n4) break;
            const float e[4] = {q[u].x, q[u].y, q[u].z, q[u].w};
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (e[k] > best.v) { best.v = e[k]; best.i = head + 4 * i4 + k; }
        }
    }
    for (int i = head + 4 * n4 + threadIdx.x; i < V; i += blockDim.x) {
        const float v = row[i];
        if (v > best.v) { best.v = v; best.i = i; }
    }
    if (best.i == 0x7fffffff && threadIdx.x == 0) best.i = 0;
    for (int off = WAVE / 2; off > 0; off >>= 1) {
        BestPair o{__shfl_xor(best.v, off, WAVE), __shfl_xor(best.i, off, WAVE)};
        best = better(best, o);
    }
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, n_waves = blockDim.x / WAVE;
    __syncthreads();
    if (lane == 0) scratch[wave] = best;
    __syncthreads();
    BestPair r = scratch[0];
    for (int w = 1; w < n_waves; ++w) r = better(r, scratch[w]);
    if (r.i == 0x7fffffff) r.i = 0;                       // a row of NaN or -inf: token 0, as the reference's loop
    return r;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void argmax_kernel(const float* __restrict__ logits, int V,
                                                                int* __restrict__ out) {
    __shared__ BestPair scratch[SAMPLE_THREADS / WAVE];
    const BestPair r = block_argmax(logits + (size_t)blockIdx.x * V, V, scratch);
    if (threadIdx.x == 0) out[blockIdx.x] = r.i;
}

PALM_API int palm_argmax(hipStream_t stream, const float* logits, int n_rows, int V, int* out) {
    PALM_CHECK(n_rows >= 0 && V > 0, "argmax: rows=%d vocab=%d", n_rows, V);
    if (n_rows == 0) return 0;
    argmax_kernel<<<n_rows, SAMPLE_THREADS, 0, stream>>>(logits, V, out);
    PALM_LAUNCHED();
    return 0;
}

// ---- penalties ------------------------------------------------------------------------------------
// One thread per (row, token, count) triple that the host has counted from the history window.
__global__ void penalties_kernel(float* __restrict__ logits, int V, const int* __restrict__ rows,
                                 const int* __restrict__ tokens, const int* __restrict__ counts, int n,
                                 float repeat_penalty, float presence, float frequency) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int tok = tokens[i];
    if (tok < 0 || tok >= V) return;
    float* p = logits + (size_t)rows[i] * V + tok;
    float l = *p;
    if (repeat_penalty != 1.0f) l = l > 0.0f ? l / repeat_penalty : l * repeat_penalty;
    l -= presence;
    l -= frequency * (float)counts[i];
    *p = l;
}

PALM_API int palm_apply_penalties(hipStream_t stream, float* logits, int V, const int* rows, const int* tokens,
                                  const int* counts, int n, float repeat_penalty, float presence, float frequency) {
    PALM_CHECK(n >= 0 && V > 0, "penalties: n=%d vocab=%d", n, V);
    PALM_CHECK(repeat_penalty > 0.f, "penalties: repeat_penalty %g must be positive", repeat_penalty);
    if (n == 0) return 0;
    penalties_kernel<<<(n + 255) / 256, 256, 0, stream>>>(logits, V, rows, tokens, counts, n, repeat_penalty,
                                                         presence, frequency);
    PALM_LAUNCHED();
    return 0;
}

// ---- sampling -------------------------------------------------------------------------------------
// Thread t owns the contiguous chunk [t * chunk, (t + 1) * chunk) of the row, so that sums and ranks
// "in index order" are a scan over threads.  All sums are added in a fixed order: the result for a row
// is the same whatever else is in the batch.

struct SampleShared {
    BestPair best[SAMPLE_THREADS / WAVE];
    float part[SAMPLE_THREADS];      // per-thread partial sums
    int cnt[SAMPLE_THREADS];         // per-thread counts
    unsigned int hist[256];
    float cand_v[TOPK_MAX];
    int cand_i[TOPK_MAX];
    float cand_w[TOPK_MAX];
    int n_cand;
    // results of the serial parts, broadcast
    uint32_t prefix; int remaining; int owner; float base; int n_ties; float total;
};

// fixed-order sum of part[0..n): a tree over the block
__device__ float block_tree_sum(float* part, int n) {
    __syncthreads();
    for (int stride = SAMPLE_THREADS / 2; stride > 0; stride >>= 1) {
        if ((int)threadIdx.x < stride && (int)threadIdx.x + stride < n) part[threadIdx.x] += part[threadIdx.x + stride];
        __syncthreads();
    }
    const float r = part[0];
    __syncthreads();
    return r;
}

// The weight of element i of the row if it is kept, else 0.  kept: key > tau, or key == tau and the
// element is among the first n_ties elements equal to tau (rank counted in index order).
__device__ inline float kept_weight(float l, float l_max, float inv_t, float min_w) {
    const float w = expf((l - l_max) * inv_t);
    return w >= min_w ? w : 0.f;
}

// Draw in index order over the kept set: the first kept element whose cumulative weight reaches target.
// `tau`/`n_ties` describe the kept set (tau == 0 keeps every key, since ordered keys of finite floats
// are > 0 ... see ordered_key: only NaN patterns could be smaller, and they carry no weight).
__device__ int draw_index_order(const float* __restrict__ row, int V, int chunk, float l_max, float inv_t,
                                float min_w, uint32_t tau, int n_ties, float target, SampleShared& sh,
                                float* __restrict__ probs_out, float total) {
    const int begin = threadIdx.x * chunk, end = min(V, begin + chunk);
    // ranks of ties: how many elements equal to tau lie before this thread's chunk
    int my_ties = 0;
    for (int i = begin; i < end; ++i) my_ties += ordered_key(row[i]) == tau;
    sh.cnt[threadIdx.x] = my_ties;
    __syncthreads();
    if (threadIdx.x == 0) {
        int run = 0;
        for (int t = 0; t < SAMPLE_THREADS; ++t) { const int c = sh.cnt[t]; sh.cnt[t] = run; run += c; }
    }
    __syncthreads();
    int tie_rank = sh.cnt[threadIdx.x];
    float mine = 0.f;
    for (int i = begin; i < end; ++i) {
        const float l = row[i];
        const uint32_t key = ordered_key(l);
        bool keep = key > tau;
        if (key == tau) { keep = tie_rank < n_ties; ++tie_rank; }
        const float w = keep ? kept_weight(l, l_max, inv_t, min_w) : 0.f;
        mine += w;
        if (probs_out) probs_out[i] = w / total;
    }
    sh.part[threadIdx.x] = mine;
    __syncthreads();
    if (threadIdx.x == 0) {
        float run = 0.f;
        int owner = -1, last_nonzero = -1;
        float base = 0.f;
        for (int t = 0; t < SAMPLE_THREADS; ++t) {
            const float p = sh.part[t];
            if (p > 0.f) last_nonzero = t;
            if (owner < 0 && p > 0.f && target <= run + p) { owner = t; base = run; }
            run += p;
        }
        // rounding can leave the target a hair above the total: then the last kept element is taken
        sh.n_ties = owner < 0;
        if (owner < 0) owner = last_nonzero;
        sh.owner = owner; sh.base = base;
    }
    __syncthreads();
    int result = -1;
    if ((int)threadIdx.x == sh.owner) {
        float run = sh.base;
        int rank = sh.cnt[threadIdx.x], last_kept = -1;
        for (int i = begin; i < end; ++i) {
            const float l = row[i];
            const uint32_t key = ordered_key(l);
            bool keep = key > tau;
            if (key == tau) { keep = rank < n_ties; ++rank; }
            const float w = keep ? kept_weight(l, l_max, inv_t, min_w) : 0.f;
            if (w > 0.f) {
                last_kept = i;
                run += w;
                if (!sh.n_ties && target <= run) { result = i; break; }
            }
        }
        if (result < 0) result = last_kept;
        sh.remaining = result;
    }
    __syncthreads();
    return sh.remaining;
}

// mass and count of the elements with key >= tau (fixed-order sums)
__device__ float mass_at_least(const float* __restrict__ row, int V, int chunk, float l_max, float inv_t,
                               float min_w, uint32_t tau, bool strict, SampleShared& sh) {
    const int begin = threadIdx.x * chunk, end = min(V, begin + chunk);
    float mine = 0.f;
    for (int i = begin; i < end; ++i) {
        const float l = row[i];
        const uint32_t key = ordered_key(l);
        if (strict ? key > tau : key >= tau) mine += kept_weight(l, l_max, inv_t, min_w);
    }
    sh.part[threadIdx.x] = mine;
    return block_tree_sum(sh.part, SAMPLE_THREADS);
}

// One block per row.  out[row] = the token; probs_out (optional, [rows, V]) = the distribution drawn from.
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, int V, const float* __restrict__ uniforms, float temperature, int top_k,
    float top_p, float min_p, int* __restrict__ out, float* __restrict__ probs_all) {
    __shared__ SampleShared sh;
    const float* row = logits + (size_t)blockIdx.x * V;
    float* probs_out = probs_all ? probs_all + (size_t)blockIdx.x * V : nullptr;
    const BestPair best = block_argmax(row, V, sh.best);
    if (temperature <= 0.f || top_k == 1) {
        if (probs_out) for (int i = threadIdx.x; i < V; i += blockDim.x) probs_out[i] = i == best.i ? 1.f : 0.f;
        if (threadIdx.x == 0) out[blockIdx.x] = best.i;
        return;
    }
    const float l_max = best.v, inv_t = 1.0f / temperature;
    const float min_w = min_p > 0.f ? min_p : 0.f;          // w_best = exp(0) = 1
    const float u = uniforms[blockIdx.x];
    const int chunk = (V + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
    const bool use_top_p = top_p > 0.f && top_p < 1.f;

    if (top_k <= 0 || top_k >= V) {
        // ---- no top-k: thresholds on the logit, draw in index order ----
        float total = mass_at_least(row, V, chunk, l_max, inv_t, min_w, 0u, false, sh);
        uint32_t tau = 0u;
        int n_ties = 0x7fffffff;
        if (use_top_p) {
            const float cutoff = top_p * total;
            // the largest tau whose mass(key >= tau) still reaches the cutoff
            uint32_t lo = 0u, hi = 0xffffffffu;              // invariant: mass(>= lo) >= cutoff
            while (lo < hi) {
                const uint32_t mid = lo + (hi - lo) / 2u + 1u;
                const float mass = mass_at_least(row, V, chunk, l_max, inv_t, min_w, mid, false, sh);
                if (mass >= cutoff) lo = mid; else hi = mid - 1u;
            }
            tau = lo;
            const float above = mass_at_least(row, V, chunk, l_max, inv_t, min_w, tau, true, sh);
            // all elements equal to tau weigh the same; take as many (in index order) as the cutoff needs
            float w_tau = 0.f;
            {
                union { uint32_t u; float f; } c;
                c.u = (tau & 0x80000000u) ? (tau & 0x7fffffffu) : ~tau;
                w_tau = kept_weight(c.f, l_max, inv_t, min_w);
            }
            n_ties = 1;
            float cum = above + w_tau;
            while (cum < cutoff && w_tau > 0.f && n_ties < V) { cum += w_tau; ++n_ties; }
            // the count of ties that exist bounds n_ties inside draw_index_order (rank < n_ties)
            total = cum;
        }
        const int tok = draw_index_order(row, V, chunk, l_max, inv_t, min_w, tau, n_ties, u * total, sh, probs_out, total);
        if (threadIdx.x == 0) out[blockIdx.x] = tok;
        return;
    }

    // ---- top-k (k <= TOPK_MAX): select, sort, then the reference's serial walk ----
    const int k = top_k;
    // radix select of the k-th largest key, 8 bits at a time from the top
    uint32_t prefix = 0u, mask = 0u;
    int remaining = k;                                       // how many of the wanted lie at or below the prefix bin
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (int i = threadIdx.x; i < 256; i += blockDim.x) sh.hist[i] = 0u;
        __syncthreads();
        for (int i = threadIdx.x; i < V; i += blockDim.x) {
            const uint32_t key = ordered_key(row[i]);
            if ((key & mask) == prefix) atomicAdd(&sh.hist[(key >> shift) & 0xffu], 1u);
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            int need = remaining;
            int bin = 255;
            for (; bin > 0; --bin) {
                const int c = (int)sh.hist[bin];
                if (c >= need) break;
                need -= c;
            }
            sh.prefix = prefix | ((uint32_t)bin << shift);
            sh.remaining = need;
        }
        __syncthreads();
        prefix = sh.prefix;
        remaining = sh.remaining;
        mask |= 0xffu << shift;
        __syncthreads();
    }
    const uint32_t tau = prefix;                             // key of the k-th largest
    const int ties_wanted = remaining;                       // how many elements equal to tau belong to the k

    // gather: everything above tau, and the first `ties_wanted` elements equal to tau in index order
    const int begin = threadIdx.x * chunk, end = min(V, begin + chunk);
    int my_ties = 0;
    for (int i = begin; i < end; ++i) my_ties += ordered_key(row[i]) == tau;
    sh.cnt[threadIdx.x] = my_ties;
    if (threadIdx.x == 0) sh.n_cand = 0;
    __syncthreads();
    if (threadIdx.x == 0) {
        int run = 0;
        for (int t = 0; t < SAMPLE_THREADS; ++t) { const int c = sh.cnt[t]; sh.cnt[t] = run; run += c; }
    }
    __syncthreads();
    {
        int rank = sh.cnt[threadIdx.x];
        for (int i = begin; i < end; ++i) {
            const float l = row[i];
            const uint32_t key = ordered_key(l);
            bool keep = key > tau;
            if (key == tau) { keep = rank < ties_wanted; ++rank; }
            if (keep) {
                const int slot = atomicAdd(&sh.n_cand, 1);
                if (slot < TOPK_MAX) { sh.cand_v[slot] = l; sh.cand_i[slot] = i; }
            }
        }
    }
    __syncthreads();
    const int n_cand = min(sh.n_cand, TOPK_MAX);
    for (int i = threadIdx.x; i < TOPK_MAX; i += blockDim.x)
        if (i >= n_cand) { sh.cand_v[i] = -INFINITY; sh.cand_i[i] = 0x7fffffff; }
    __syncthreads();
    // bitonic sort by (value descending, index ascending)
    for (int size = 2; size <= TOPK_MAX; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            const int i = threadIdx.x;
            const int j = i ^ stride;
            if (j > i && i < TOPK_MAX) {
                const bool descending = (i & size) == 0;
                const float vi = sh.cand_v[i], vj = sh.cand_v[j];
                const int ii = sh.cand_i[i], ij = sh.cand_i[j];
                const bool i_first = vi > vj || (vi == vj && ii < ij);   // i belongs before j in the final order
                if (i_first != descending) {
                    sh.cand_v[i] = vj; sh.cand_v[j] = vi;
                    sh.cand_i[i] = ij; sh.cand_i[j] = ii;
                }
            }
            __syncthreads();
        }
    }
    for (int i = threadIdx.x; i < n_cand; i += blockDim.x) sh.cand_w[i] = expf((sh.cand_v[i] - l_max) * inv_t);
    if (probs_out) for (int i = threadIdx.x; i < V; i += blockDim.x) probs_out[i] = 0.f;
    __syncthreads();
    if (threadIdx.x == 0) {
        // engine/sampler.cpp:126-157 and :180-187, in the same order of operations
        int active = n_cand;
        if (min_p > 0.f) {
            const float threshold = min_p * sh.cand_w[0];
            active = 1;
            while (active < n_cand && sh.cand_w[active] >= threshold) ++active;
        }
        float sum = 0.f;
        for (int i = 0; i < active; ++i) sum += sh.cand_w[i];
        if (!(sum > 0.f) || !isfinite(sum)) { sh.cand_w[0] = 1.f; active = 1; sum = 1.f; }
        if (use_top_p) {
            const float cutoff = top_p * sum;
            float cum = 0.f;
            for (int i = 0; i < active; ++i) {
                cum += sh.cand_w[i];
                if (cum >= cutoff) { active = i + 1; sum = cum; break; }
            }
        }
        const float target = u * sum;
        float cum = 0.f;
        int pick = sh.cand_i[active - 1];
        for (int i = 0; i < active; ++i) {
            cum += sh.cand_w[i];
            if (target <= cum) { pick = sh.cand_i[i]; break; }
        }
        out[blockIdx.x] = pick;
        sh.remaining = active;
        sh.total = sum;
    }
    __syncthreads();
    if (probs_out) {
        __threadfence_block();
        for (int i = threadIdx.x; i < sh.remaining; i += blockDim.x) probs_out[sh.cand_i[i]] = sh.cand_w[i] / sh.total;
    }
}

PALM_API int palm_sample(hipStream_t stream, const float* logits, int n_rows, int V, const float* uniforms,
                         float temperature, int top_k, float top_p, float min_p, int* out, float* probs_out) {
    PALM_CHECK(n_rows >= 0 && V > 0, "sample: rows=%d vocab=%d", n_rows, V);
    PALM_CHECK(temperature >= 0.f && temperature <= 2.f, "sample: temperature must be between 0 and 2");
    PALM_CHECK(top_k >= 0, "sample: top_k must be non-negative");
    PALM_CHECK(top_p >= 0.f && top_p <= 1.f, "sample: top_p must be between 0 and 1");
    PALM_CHECK(min_p >= 0.f && min_p <= 1.f, "sample: min_p must be between 0 and 1");
    PALM_CHECK(top_k <= TOPK_MAX || top_k >= V, "sample: top_k = %d; this kernel sorts at most %d candidates "
               "(use 0 to switch top-k off)", top_k, TOPK_MAX);
    PALM_CHECK(temperature <= 0.f || top_k == 1 || uniforms, "sample: a draw needs the uniform numbers");
    if (n_rows == 0) return 0;
    sample_kernel<<<n_rows, SAMPLE_THREADS, 0, stream>>>(logits, V, uniforms, temperature, top_k, top_p, min_p, out,
                                                        probs_out);
    PALM_LAUNCHED();
    return 0;
}
