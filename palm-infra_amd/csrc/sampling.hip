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
// One block of 16 waves for each row.  Wave w owns the contiguous range [w * per, (w + 1) * per) of the row and
// walks it 64 elements at a time, a lane an element: reads are contiguous, and "index order" is the order
// (wave, step, lane).  A weight is w = exp((l - l_max) / T), at most 1; sums of weights are 64-bit sums of the
// integers floor(w * 2^31).  Integer sums do not depend on the order of their terms: a row's result is the same
// bits whatever else is in the batch, however the atomic additions below fall, and a part's sum is exactly the
// sum of its parts' (so a search that goes from waves to threads to elements never misses its target).

constexpr int SAMPLE_WAVES = SAMPLE_THREADS / WAVE;
constexpr float FIXED_ONE = 2147483648.0f;           // 2^31: a weight fits 32 bits, a row's sum 64
constexpr int HIST_STRIDE = 257;                     // a wave's histogram starts one bank on from its neighbour's
constexpr int SEG_CAP = 256;                         // elements a wave can set aside for the later passes of top-k
constexpr int COARSE_BINS = 1024;
static_assert(COARSE_BINS == SAMPLE_THREADS, "a thread a bin in the scan over the bins");

// 0 for the row's maximum, growing with the distance below it: 64 bins for each doubling of (distance + 1), so
// the few elements near the top have bins to themselves, and the many far below still spread over some dozen bins
// (additions to one bin take turns).  Monotone: an element in a lower bin is at least as large as one in a higher.
__device__ inline int coarse_bin(float l, float l_max) {
    const float f = (l_max - l) + 1.0f;                        // at least 1, or NaN
    const uint32_t b = (__float_as_uint(f) - 0x3f800000u) >> 17;
    return f >= 1.0f ? (int)min(b, (uint32_t)COARSE_BINS - 1u) : COARSE_BINS - 1;
}
typedef unsigned long long mass_t;

struct SampleShared {
    BestPair best[SAMPLE_WAVES];
    union {
        mass_t mass[SAMPLE_WAVES][HIST_STRIDE];          // a histogram for each wave: weights by a byte of the key
        unsigned int count[SAMPLE_WAVES][HIST_STRIDE];   //                            elements by a byte of the key
        struct {                                         // or: the few elements still in the running, by wave
            uint32_t key[SAMPLE_WAVES][SEG_CAP];
            int idx[SAMPLE_WAVES][SEG_CAP];
        } seg;
    } hist;
    unsigned int small[256];                     // one histogram for the block, where few elements are counted
    union {                                      // by the distance below the maximum:
        unsigned int coarse[COARSE_BINS];        //   elements (top-k)
        mass_t coarse_mass[COARSE_BINS];         //   weights (top-p)
    };
    mass_t bin_mass[256];
    mass_t wave_mass[SAMPLE_WAVES];              // weights above the threshold, by wave; then by wave of threads
    int wave_ties[SAMPLE_WAVES];                 // elements at the threshold
    float cand_v[TOPK_MAX];
    int cand_i[TOPK_MAX];
    float cand_w[TOPK_MAX];
    int n_cand;
    // results of the serial parts, broadcast
    uint32_t prefix; int remaining; int owner; int owner_ties; mass_t base; mass_t above; float total; int result;
};

__device__ inline uint32_t fixed_weight(float l, float l_max, float inv_t, float min_w) {
    const float w = __expf((l - l_max) * inv_t);
    return w >= min_w ? (uint32_t)(w * FIXED_ONE) : 0u;       // (a NaN fails the comparison)
}
__device__ inline float key_value(uint32_t key) {             // the float whose ordered_key is key
    return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}
__device__ inline mass_t wave_sum(mass_t v) {
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, WAVE);
    return v;
}
__device__ inline int wave_sum(int v) {
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, WAVE);
    return v;
}
// how many lanes below this one have the flag set
__device__ inline int lanes_before(bool flag) {
    const unsigned long long m = __ballot(flag);
    return __popcll(m & ((1ull << (threadIdx.x % WAVE)) - 1ull));
}

// The wave's range of the row, and f(i, l) for its elements in index order (every lane takes part in every
// step; a lane beyond the range gets i = -1 and l = -inf).
struct Range { int begin, end; };
__device__ inline Range wave_range(int V) {
    const int per = ((V + SAMPLE_WAVES - 1) / SAMPLE_WAVES + WAVE - 1) / WAVE * WAVE;
    const int begin = min(V, (int)(threadIdx.x / WAVE) * per);
    return Range{begin, min(V, begin + per)};
}
constexpr int RANGE_AHEAD = 16;          // steps whose reads are on their way together: the row comes from L2, a read takes long
template <typename F>
__device__ inline void for_range(const float* __restrict__ row, Range rg, F&& f) {
    const int lane = threadIdx.x % WAVE;
    for (int base = rg.begin; base < rg.end; base += RANGE_AHEAD * WAVE) {
        float l[RANGE_AHEAD];
#pragma unroll
        for (int u = 0; u < RANGE_AHEAD; ++u) {
            const int i = base + u * WAVE + lane;
            l[u] = i < rg.end ? row[i] : -INFINITY;
        }
#pragma unroll
        for (int u = 0; u < RANGE_AHEAD; ++u) {
            const int i = base + u * WAVE + lane;
            if (base + u * WAVE < rg.end) f(i < rg.end ? i : -1, l[u]);
        }
    }
}

// wave_mass[w] = the weights of wave w's elements with key > tau (all of them if `all`), wave_ties[w] = how many
// of its elements have key == tau; then a barrier
template <bool WEIGHTS = true>     // false: wave_mass[w] counts the elements instead of weighing them
__device__ void masses_by_wave(const float* __restrict__ row, int V, float l_max, float inv_t, float min_w, uint32_t tau,
                               bool all, SampleShared& sh) {
    mass_t mine = 0ull;
    int ties = 0;
    for_range(row, wave_range(V), [&](int i, float l) {
        const uint32_t key = ordered_key(l);
        if (i >= 0 && (all || key > tau)) mine += WEIGHTS ? fixed_weight(l, l_max, inv_t, min_w) : 1u;
        ties += i >= 0 && !all && key == tau;
    });
    mine = wave_sum(mine);
    ties = wave_sum(ties);
    if (threadIdx.x % WAVE == 0) { sh.wave_mass[threadIdx.x / WAVE] = mine; sh.wave_ties[threadIdx.x / WAVE] = ties; }
    __syncthreads();
}

// The element in which the weights of the kept set, added up in index order, pass `target` (< their sum).
// The kept set: key > tau, and the first n_ties elements with key == tau (`all`: every element).  Needs
// masses_by_wave(tau).  Three levels: the wave's range, a thread's piece of that range, the element.
__device__ int draw_index_order(const float* __restrict__ row, int V, float l_max, float inv_t, float min_w, uint32_t tau,
                                bool all, int n_ties, mass_t w_tau, mass_t target, SampleShared& sh) {
    if (threadIdx.x == 0) {
        mass_t run = 0ull;
        int ties_before = 0, owner = SAMPLE_WAVES - 1, owner_ties = 0;
        mass_t base = 0ull;
        bool found = false;
        for (int w = 0; w < SAMPLE_WAVES; ++w) {
            const int kept_ties = all ? 0 : max(0, min(sh.wave_ties[w], n_ties - ties_before));
            const mass_t kept = sh.wave_mass[w] + (mass_t)kept_ties * w_tau;
            if (!found && target < run + kept) { found = true; owner = w; base = run; owner_ties = ties_before; }
            run += kept;
            ties_before += sh.wave_ties[w];
        }
        sh.owner = owner; sh.base = base; sh.owner_ties = owner_ties;
    }
    __syncthreads();
    // the owner's range, a piece a thread
    const int per = ((V + SAMPLE_WAVES - 1) / SAMPLE_WAVES + WAVE - 1) / WAVE * WAVE;
    const int r_begin = min(V, sh.owner * per), r_end = min(V, r_begin + per);
    const int piece = (r_end - r_begin + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
    const int begin = min(r_end, r_begin + (int)threadIdx.x * piece), end = min(r_end, begin + piece);
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    mass_t above = 0ull;
    int ties = 0;
    for (int i = begin; i < end; ++i) {
        const float l = row[i];
        const uint32_t key = ordered_key(l);
        if (all || key > tau) above += fixed_weight(l, l_max, inv_t, min_w);
        ties += !all && key == tau;
    }
    // ties before this thread's piece: a scan over the lanes, then over the waves
    int tie_scan = ties;
#pragma unroll
    for (int off = 1; off < WAVE; off <<= 1) { const int o = __shfl_up(tie_scan, off, WAVE); if (lane >= off) tie_scan += o; }
    if (lane == WAVE - 1) sh.wave_ties[wave] = tie_scan;
    __syncthreads();
    int ties_before = sh.owner_ties + tie_scan - ties;
    for (int w = 0; w < wave; ++w) ties_before += sh.wave_ties[w];
    const int kept_ties = all ? 0 : max(0, min(ties, n_ties - ties_before));
    const mass_t kept = above + (mass_t)kept_ties * w_tau;
    mass_t scan = kept;
#pragma unroll
    for (int off = 1; off < WAVE; off <<= 1) { const mass_t o = __shfl_up(scan, off, WAVE); if (lane >= off) scan += o; }
    if (lane == WAVE - 1) sh.wave_mass[wave] = scan;
    if (threadIdx.x == 0) sh.result = -1;
    __syncthreads();
    mass_t before = sh.base + scan - kept;
    for (int w = 0; w < wave; ++w) before += sh.wave_mass[w];
    if (target >= before && target < before + kept) {          // one thread at most: the pieces' sums tile the range's
        mass_t run = before;
        int rank = ties_before;
        for (int i = begin; i < end; ++i) {
            const float l = row[i];
            const uint32_t key = ordered_key(l);
            bool keep = all || key > tau;
            if (!all && key == tau) { keep = rank < n_ties; ++rank; }
            if (keep) {
                run += fixed_weight(l, l_max, inv_t, min_w);
                if (target < run) { sh.result = i; break; }
            }
        }
    }
    __syncthreads();
    return sh.result;
}

// probs_out[i] = the element's share of the kept set's weight (needs masses_by_wave(tau) for the ties' ranks)
__device__ void write_probabilities(const float* __restrict__ row, int V, float l_max, float inv_t, float min_w, uint32_t tau,
                                    bool all, int n_ties, mass_t total, const SampleShared& sh, float* __restrict__ probs_out) {
    int rank = 0;
    for (int w = 0; w < (int)(threadIdx.x / WAVE); ++w) rank += sh.wave_ties[w];
    const float inv_total = 1.0f / (float)total;
    for_range(row, wave_range(V), [&](int i, float l) {
        const uint32_t key = ordered_key(l);
        const bool tie = i >= 0 && !all && key == tau;
        bool keep = i >= 0 && (all || key > tau);
        const int before = lanes_before(tie);
        if (tie) keep = rank + before < n_ties;
        rank += __popcll(__ballot(tie));
        if (i >= 0) probs_out[i] = keep ? (float)fixed_weight(l, l_max, inv_t, min_w) * inv_total : 0.f;
    });
}

// One block per row.  out[row] = the token; probs_out (optional, [rows, V]) = the distribution drawn from.
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, int V, const float* __restrict__ uniforms, float temperature, int top_k,
    float top_p, float min_p, int* __restrict__ out, float* __restrict__ probs_all) {
    __shared__ SampleShared sh;
    const float* row = logits + (size_t)blockIdx.x * V;
    float* probs_out = probs_all ? probs_all + (size_t)blockIdx.x * V : nullptr;
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    const BestPair best = block_argmax(row, V, sh.best);
    if (temperature <= 0.f || top_k == 1) {
        if (probs_out) for (int i = threadIdx.x; i < V; i += blockDim.x) probs_out[i] = i == best.i ? 1.f : 0.f;
        if (threadIdx.x == 0) out[blockIdx.x] = best.i;
        return;
    }
    const float l_max = best.v, inv_t = 1.0f / temperature;
    const float min_w = min_p > 0.f ? min_p : 0.f;          // w_best = exp(0) = 1
    const float u = uniforms[blockIdx.x];
    const bool use_top_p = top_p > 0.f && top_p < 1.f;
    const Range mine = wave_range(V);

    if (top_k <= 0 || top_k >= V) {
        // ---- no top-k: a threshold on the logit, the draw in index order ----
        // the weight of the whole row: by wave for the draw, or (top-p, which first looks for its threshold) by distance
        // below the maximum, see below
        const bool coarse_first = use_top_p && !probs_out;
        mass_t total = 0ull;
        if (coarse_first) {
            sh.coarse_mass[threadIdx.x] = 0ull;
            __syncthreads();
            for_range(row, mine, [&](int i, float l) {
                const uint32_t w = i >= 0 ? fixed_weight(l, l_max, inv_t, min_w) : 0u;
                if (w) atomicAdd(&sh.coarse_mass[coarse_bin(l, l_max)], (mass_t)w);
            });
            __syncthreads();
            mass_t part = 0ull;
            for (int b = lane; b < COARSE_BINS; b += WAVE) part += sh.coarse_mass[b];
            total = wave_sum(part);
        } else {
            masses_by_wave(row, V, l_max, inv_t, min_w, 0u, true, sh);
            for (int w = 0; w < SAMPLE_WAVES; ++w) total += sh.wave_mass[w];
        }
        if (total == 0ull) {                                 // nothing has weight (a row of -inf or NaN): the first maximum
            if (probs_out) for (int i = threadIdx.x; i < V; i += blockDim.x) probs_out[i] = i == best.i ? 1.f : 0.f;
            if (threadIdx.x == 0) out[blockIdx.x] = best.i;
            return;
        }
        uint32_t tau = 0u;
        bool all = true;
        int n_ties = 0;
        mass_t w_tau = 0ull;
        if (use_top_p) {
            // The largest tau whose elements with key >= tau weigh at least the cutoff, a byte of the key at a time
            // from the top: the weights of the elements that match the bytes found so far, by their next byte.
            mass_t cutoff = (mass_t)((double)top_p * (double)total);
            if (cutoff < 1ull) cutoff = 1ull;
            uint32_t prefix = 0u, mask = 0u;
            mass_t above = 0ull;                             // the weight of the keys above the bytes found so far
            __syncthreads();
            // First a coarse cut, as for top-k: the weights by their distance below the maximum (added up above), the bin in
            // which they reach the cutoff, the elements of the bins up to it set aside.  If they fit, the threshold, the
            // ties and the draw are found among them.  (The probabilities are written from the row: not here.)
            if (coarse_first) {
                const mass_t mine_m = sh.coarse_mass[threadIdx.x];
                mass_t scan = mine_m;
#pragma unroll
                for (int off = 1; off < WAVE; off <<= 1) { const mass_t o = __shfl_up(scan, off, WAVE); if (lane >= off) scan += o; }
                if (lane == WAVE - 1) sh.wave_mass[wave] = scan;
                if (threadIdx.x == 0) sh.owner = COARSE_BINS - 1;
                __syncthreads();
                for (int w = 0; w < wave; ++w) scan += sh.wave_mass[w];
                if (scan - mine_m < cutoff && cutoff <= scan) sh.owner = threadIdx.x;
                __syncthreads();
                const int cut = sh.owner;
                // How many elements that is at least: a bin's weight over the largest weight an element of it can
                // have.  A flat row keeps most of its elements; then setting them aside is a pass for nothing.
                if (threadIdx.x == 0) sh.n_cand = 0;
                __syncthreads();
                if ((int)threadIdx.x <= cut && mine_m) {
                    const float nearest = __uint_as_float(((uint32_t)threadIdx.x << 17) + 0x3f800000u) - 1.0f;   // coarse_bin, backwards
                    const mass_t heaviest = (mass_t)fixed_weight(l_max - nearest, l_max, inv_t, 0.f) + 1ull;
                    atomicAdd(&sh.n_cand, (int)min(mine_m / heaviest, (mass_t)(1 << 20)));
                }
                __syncthreads();
                bool fits = sh.n_cand <= SEG_CAP * SAMPLE_WAVES;
                int seg_n = 0;
                if (fits) {
                    for_range(row, mine, [&](int i, float l) {
                        const bool match = i >= 0 && coarse_bin(l, l_max) <= cut;
                        const int at = seg_n + lanes_before(match);
                        if (match && at < SEG_CAP) { sh.hist.seg.key[wave][at] = ordered_key(l); sh.hist.seg.idx[wave][at] = i; }
                        seg_n += __popcll(__ballot(match));
                    });
                    if (lane == 0) sh.wave_ties[wave] = seg_n;
                    __syncthreads();
                    for (int w = 0; w < SAMPLE_WAVES; ++w) fits = fits && sh.wave_ties[w] <= SEG_CAP;
                    __syncthreads();
                }
                if (fits) {
                    // f(key, index) for the wave's elements set aside, in index order; every lane takes part in every step
                    auto each = [&](auto&& f) {
                        for (int j0 = 0; j0 < seg_n; j0 += WAVE) {
                            const bool valid = j0 + lane < seg_n;
                            f(valid ? sh.hist.seg.key[wave][j0 + lane] : 0u, valid ? sh.hist.seg.idx[wave][j0 + lane] : -1);
                        }
                    };
                    for (int shift = 24; shift >= 0; shift -= 8) {
                        if (threadIdx.x < 256) sh.bin_mass[threadIdx.x] = 0ull;
                        __syncthreads();
                        each([&](uint32_t key, int i) {
                            if (i >= 0 && (key & mask) == prefix) {
                                const uint32_t w = fixed_weight(key_value(key), l_max, inv_t, min_w);
                                if (w) atomicAdd(&sh.bin_mass[(key >> shift) & 0xffu], (mass_t)w);
                            }
                        });
                        __syncthreads();
                        if (threadIdx.x == 0) {
                            mass_t run = above;
                            int bin = 255;
                            for (; bin > 0; --bin) {
                                if (run + sh.bin_mass[bin] >= cutoff) break;
                                run += sh.bin_mass[bin];
                            }
                            sh.prefix = prefix | ((uint32_t)bin << shift);
                            sh.above = run;
                        }
                        __syncthreads();
                        prefix = sh.prefix;
                        above = sh.above;
                        mask |= 0xffu << shift;
                    }
                    tau = prefix;
                    w_tau = (mass_t)fixed_weight(key_value(tau), l_max, inv_t, min_w);
                    n_ties = w_tau ? (int)min((mass_t)V, (cutoff - above + w_tau - 1ull) / w_tau) : 0;
                    total = above + (mass_t)n_ties * w_tau;
                    mass_t target = (mass_t)((double)u * (double)total);
                    if (target >= total) target = total - 1ull;
                    // the kept weights by wave, then the wave in which they pass the target, then the element
                    mass_t kept = 0ull;
                    int ties = 0;
                    each([&](uint32_t key, int i) {
                        if (i >= 0 && key > tau) kept += fixed_weight(key_value(key), l_max, inv_t, min_w);
                        ties += i >= 0 && key == tau;
                    });
                    kept = wave_sum(kept);
                    ties = wave_sum(ties);
                    if (lane == 0) { sh.wave_mass[wave] = kept; sh.wave_ties[wave] = ties; }
                    if (threadIdx.x == 0) sh.result = -1;
                    __syncthreads();
                    mass_t before = 0ull;
                    int ties_before = 0;
                    for (int w = 0; w < wave; ++w) {
                        before += sh.wave_mass[w] + (mass_t)max(0, min(sh.wave_ties[w], n_ties - ties_before)) * w_tau;
                        ties_before += sh.wave_ties[w];
                    }
                    const mass_t here = kept + (mass_t)max(0, min(ties, n_ties - ties_before)) * w_tau;
                    if (target >= before && target < before + here) {        // one wave at most
                        mass_t run = before;
                        int rank = ties_before;
                        bool found = false;
                        each([&](uint32_t key, int i) {
                            const bool tie = i >= 0 && key == tau;
                            bool keep = i >= 0 && key > tau;
                            const int at = rank + lanes_before(tie);
                            if (tie) keep = at < n_ties;
                            rank += __popcll(__ballot(tie));
                            const mass_t w = keep ? (mass_t)fixed_weight(key_value(key), l_max, inv_t, min_w) : 0ull;
                            mass_t scan = w;
#pragma unroll
                            for (int off = 1; off < WAVE; off <<= 1) { const mass_t o = __shfl_up(scan, off, WAVE); if (lane >= off) scan += o; }
                            const unsigned long long hit = __ballot(w > 0ull && target < run + scan);
                            if (!found && hit) {
                                found = true;
                                if (lane == __ffsll((long long)hit) - 1) sh.result = i;
                            }
                            run += __shfl(scan, WAVE - 1, WAVE);
                        });
                    }
                    __syncthreads();
                    if (threadIdx.x == 0) out[blockIdx.x] = sh.result >= 0 ? sh.result : best.i;
                    return;
                }
            }
            // The top byte of a float's key is its sign and most of its exponent: most of a row shares one or two
            // values of it, and as many additions to one histogram bin take as many turns.  Usually the elements
            // that share the maximum's top byte already weigh as much as the cutoff: then that byte is the answer.
            const uint32_t top = ordered_key(l_max) & 0xff000000u;
            int first_shift = 24;
            if (top) {
                masses_by_wave(row, V, l_max, inv_t, min_w, top - 1u, false, sh);
                mass_t with_top = 0ull;
                for (int w = 0; w < SAMPLE_WAVES; ++w) with_top += sh.wave_mass[w];
                if (with_top >= cutoff) { prefix = top; mask = 0xff000000u; first_shift = 16; }
                __syncthreads();
            }
            for (int shift = first_shift; shift >= 0; shift -= 8) {
                for (int i = threadIdx.x; i < SAMPLE_WAVES * HIST_STRIDE; i += blockDim.x) (&sh.hist.mass[0][0])[i] = 0ull;
                __syncthreads();
                for_range(row, mine, [&](int i, float l) {
                    const uint32_t key = ordered_key(l);
                    const uint32_t w = i >= 0 && (key & mask) == prefix ? fixed_weight(l, l_max, inv_t, min_w) : 0u;
                    const int bin = w ? (int)((key >> shift) & 0xffu) : -1;
                    if (bin >= 0) atomicAdd(&sh.hist.mass[wave][bin], (mass_t)w);
                });
                __syncthreads();
                if (threadIdx.x < 256) {
                    mass_t sum = 0ull;
                    for (int w = 0; w < SAMPLE_WAVES; ++w) sum += sh.hist.mass[w][threadIdx.x];
                    sh.bin_mass[threadIdx.x] = sum;
                }
                __syncthreads();
                if (threadIdx.x == 0) {
                    mass_t run = above;
                    int bin = 255;
                    for (; bin > 0; --bin) {
                        if (run + sh.bin_mass[bin] >= cutoff) break;
                        run += sh.bin_mass[bin];
                    }
                    sh.prefix = prefix | ((uint32_t)bin << shift);
                    sh.above = run;
                }
                __syncthreads();
                prefix = sh.prefix;
                above = sh.above;
                mask |= 0xffu << shift;
            }
            tau = prefix;
            all = false;
            // the elements equal to tau weigh the same; as many of them (in index order) as the cutoff needs
            w_tau = (mass_t)fixed_weight(key_value(tau), l_max, inv_t, min_w);
            n_ties = w_tau ? (int)min((mass_t)V, (cutoff - above + w_tau - 1ull) / w_tau) : 0;
            total = above + (mass_t)n_ties * w_tau;
            masses_by_wave(row, V, l_max, inv_t, min_w, tau, false, sh);
        }
        mass_t target = (mass_t)((double)u * (double)total);
        if (target >= total) target = total - 1ull;
        if (probs_out) write_probabilities(row, V, l_max, inv_t, min_w, tau, all, n_ties, total, sh, probs_out);
        const int tok = draw_index_order(row, V, l_max, inv_t, min_w, tau, all, n_ties, w_tau, target, sh);
        if (threadIdx.x == 0) out[blockIdx.x] = tok >= 0 ? tok : best.i;
        return;
    }

    // ---- top-k (k <= TOPK_MAX): select, sort, then the reference's serial walk ----
    const int k = top_k;
    // the key of the k-th largest element, a byte at a time from the top: how many of the elements that match the
    // bytes found so far have which next byte
    uint32_t prefix = 0u, mask = 0u;
    int remaining = k;                                       // how many of the wanted lie at or below the prefix bin
    // First a coarse cut: count the elements by their distance below the maximum, find the bin in which the k-th
    // largest lies, and set the elements of the bins up to it aside, by wave and in index order.  If every wave's
    // fit, the exact search and the gathering walk them instead of the row.
    int seg_n = 0;
    bool compact = false;
    {
        sh.coarse[threadIdx.x] = 0u;
        __syncthreads();
        for_range(row, mine, [&](int i, float l) { if (i >= 0) atomicAdd(&sh.coarse[coarse_bin(l, best.v)], 1u); });
        __syncthreads();
        // a scan over the bins, a thread a bin: the bin where the running count reaches k
        const int mine_c = (int)sh.coarse[threadIdx.x];
        int scan = mine_c;
#pragma unroll
        for (int off = 1; off < WAVE; off <<= 1) { const int o = __shfl_up(scan, off, WAVE); if (lane >= off) scan += o; }
        if (lane == WAVE - 1) sh.wave_ties[wave] = scan;
        if (threadIdx.x == 0) sh.owner = COARSE_BINS - 1;
        __syncthreads();
        for (int w = 0; w < wave; ++w) scan += sh.wave_ties[w];
        if (scan - mine_c < k && k <= scan) sh.owner = threadIdx.x;
        __syncthreads();
        const int cut = sh.owner;
        int n = 0;
        for_range(row, mine, [&](int i, float l) {
            const bool match = i >= 0 && coarse_bin(l, best.v) <= cut;
            const int at = n + lanes_before(match);
            if (match && at < SEG_CAP) { sh.hist.seg.key[wave][at] = ordered_key(l); sh.hist.seg.idx[wave][at] = i; }
            n += __popcll(__ballot(match));
        });
        __syncthreads();                                     // (wave_ties is read above)
        if (lane == 0) sh.wave_ties[wave] = n;
        __syncthreads();
        bool fits = true;
        for (int w = 0; w < SAMPLE_WAVES; ++w) fits = fits && sh.wave_ties[w] <= SEG_CAP;
        compact = fits;
        seg_n = compact ? n : 0;
        __syncthreads();
    }
    const int first_shift = 24;
    // f(i, l) for the elements in the running, in index order within the wave
    auto each = [&](auto&& f) {
        if (compact) {
            for (int j0 = 0; j0 < seg_n; j0 += WAVE) {
                const bool valid = j0 + lane < seg_n;
                f(valid ? sh.hist.seg.idx[wave][j0 + lane] : -1, valid ? key_value(sh.hist.seg.key[wave][j0 + lane]) : -INFINITY);
            }
        } else {
            for_range(row, mine, f);
        }
    };
    for (int shift = first_shift; shift >= 0; shift -= 8) {
        if (compact) { if (threadIdx.x < 256) sh.small[threadIdx.x] = 0u; }
        else for (int i = threadIdx.x; i < SAMPLE_WAVES * HIST_STRIDE; i += blockDim.x) (&sh.hist.count[0][0])[i] = 0u;
        __syncthreads();
        each([&](int i, float l) {
            const uint32_t key = ordered_key(l);
            const int bin = i >= 0 && (key & mask) == prefix ? (int)((key >> shift) & 0xffu) : -1;
            if (bin >= 0) atomicAdd(compact ? &sh.small[bin] : &sh.hist.count[wave][bin], 1u);
        });
        __syncthreads();
        if (threadIdx.x < 256) {
            unsigned int sum = 0u;
            if (compact) sum = sh.small[threadIdx.x];
            else for (int w = 0; w < SAMPLE_WAVES; ++w) sum += sh.hist.count[w][threadIdx.x];
            sh.bin_mass[threadIdx.x] = sum;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            int need = remaining;
            int bin = 255;
            for (; bin > 0; --bin) {
                const int c = (int)sh.bin_mass[bin];
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
    }
    const uint32_t tau = prefix;                             // key of the k-th largest
    const int ties_wanted = remaining;                       // how many elements equal to tau belong to the k

    // gather: everything above tau, and the first `ties_wanted` elements equal to tau in index order
    {
        int rank = 0;
        if (compact) {
            int ties = 0;
            each([&](int i, float l) { ties += i >= 0 && ordered_key(l) == tau; });
            ties = wave_sum(ties);
            if (lane == 0) sh.wave_ties[wave] = ties;
            __syncthreads();
            for (int w = 0; w < wave; ++w) rank += sh.wave_ties[w];
        } else {                                             // the last histogram holds each wave's count of them
            for (int w = 0; w < wave; ++w) rank += (int)sh.hist.count[w][tau & 0xffu];
        }
        if (threadIdx.x == 0) sh.n_cand = 0;
        __syncthreads();
        each([&](int i, float l) {
            const uint32_t key = ordered_key(l);
            const bool tie = i >= 0 && key == tau;
            bool keep = i >= 0 && key > tau;
            const int before = lanes_before(tie);
            if (tie) keep = rank + before < ties_wanted;
            rank += __popcll(__ballot(tie));
            if (keep) {
                const int slot = atomicAdd(&sh.n_cand, 1);
                if (slot < TOPK_MAX) { sh.cand_v[slot] = l; sh.cand_i[slot] = i; }
            }
        });
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
