// Causal grouped-query attention over the paged cache on the matrix cores, bfloat16, compiled for one
// head size (PALM_HEAD_DIM, a multiple of 16).  Same semantics as the exact kernel
// (models/qwen3.py:336-341; kernels/attention.cpp:84-217, 937-962): head h reads kv head h / (nh / nkv),
// keys j <= p of the query's own sequence (j > p - window with a window), softmax in 32-bit with the
// running maximum, o = sum_j p_j v_j.
//
// Cache layouts: K [pages, nkv, 64 keys, hd] (a key's row is contiguous); V is kept transposed,
// [pages, nkv, hd, 64 keys], so that for both products the summed index is contiguous in memory.
//
// Formulation (transposed, so that no operand has to be shuffled between the two products):
//   S^T[key, query] = sum_d K[key, d] Q[query, d]        A = K rows, B = Q rows
//   O^T[d, query]   = sum_key V^T[d, key] P^T[key, query]  A = V^T rows, B = P^T = the registers S^T left
// A 16x16 result tile leaves lane (q, g) with rows 4g..4g+3 of column q.  Two S^T tiles therefore give a
// lane eight keys of one query, which is exactly a B operand of the second product if the tiles' rows are
// chosen as keys {8g'+0..3} and {8g'+4..7} of a run of 32 keys: then the eight keys of lane group g are
// keys 8g..8g+7, one 16-byte read of a V^T row.  All softmax statistics are per column, i.e. per lane.
//
// decode:  one wave per (sequence, kv head, slice of the key range); the G = nh / nkv query heads of the
//          kv head are the columns.  Partial (max, sum, output) go to a workspace and a second kernel
//          merges the slices.  The kernel is bound by reading K and V once.
// prefill: one block of four waves per (sequence, kv head, 16 query positions); wave w owns the columns
//          of query head w of the group (more heads: more passes).
#include <mutex>

#include "mfma.h"
#include "attention_api.h"

#ifndef PALM_HEAD_DIM
#error "compile with -DPALM_HEAD_DIM=<head size>"
#endif

constexpr int HD = PALM_HEAD_DIM;
static_assert(HD % 16 == 0 && HD >= 16 && HD <= 256, "head size must be a multiple of 16, at most 256");
constexpr int CHUNKS = HD / 8;               // 16-byte chunks in a row of K or Q
constexpr int KSTEPS = (CHUNKS + 3) / 4;     // MFMA steps over d (32 values each; the last may be half empty)
constexpr int DTILES = HD / 16;              // 16-row tiles of O^T
constexpr float LOG2E = 1.4426950408889634f;

// 2^x as the one hardware instruction.  The library's exp2f wraps it in a rescaling so that results below
// 2^-126 come out as denormals; a softmax weight that small adds nothing to a sum whose largest term is 1, and
// the wrapper costs a quarter of the kernel's vector instructions.  Arguments here are <= 0 (or -inf, giving 0).
__device__ inline float exp2_weight(float x) { return __builtin_amdgcn_exp2f(x); }

PALM_DEFINE_LAST_ERROR()
PALM_API int palm_attention_head_dim() { return HD; }
PALM_API int palm_attention_page_tokens() { return PAGE_TOKENS; }

struct Columns {          // softmax state of this lane's query column, and its share of the output
    float m, l;
    f32x4 o[DTILES];
};

// The key that row r of S^T tile `t` (0..3) of a page stands for: tiles 2h and 2h+1 cover keys 32h..32h+31.
__device__ inline int tile_key(int t, int r) { return (t / 2) * 32 + (r / 4) * 8 + (t % 2) * 4 + (r % 4); }

// The operands of one page, read ahead of their use: K fragments for the first product, V^T fragments for
// the second.  Every read is unconditional (an absent chunk reads chunk 0 and is zeroed by a select), so the
// compiler can issue them all before the first wait; a read behind a branch would be waited for one by one.
struct PageOperands {
    bf16x8 k[4][KSTEPS];
    bf16x8 v[DTILES][2];
};

__device__ inline void load_keys(const bf16_t* __restrict__ kp, int r, int g, PageOperands& ops) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const bf16_t* krow = kp + (size_t)tile_key(t, r) * HD;
#pragma unroll
        for (int j = 0; j < KSTEPS; ++j) {
            const int chunk = j * 4 + g;
            const bool ok = (CHUNKS % 4 == 0) || chunk < CHUNKS;
            const bf16x8 v = load_bf16x8(krow + (ok ? chunk : 0) * 8);
            ops.k[t][j] = ok ? v : zero_bf16x8();
        }
    }
}

__device__ inline void load_values(const bf16_t* __restrict__ vp, int r, int g, PageOperands& ops) {
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) {
        const bf16_t* vrow = vp + (size_t)(dt * 16 + r) * PAGE_TOKENS;
#pragma unroll
        for (int h = 0; h < 2; ++h) ops.v[dt][h] = load_bf16x8(vrow + h * 32 + g * 8);
    }
}

// Scores of a page's 64 keys against the columns' queries and the online softmax; leaves the page's
// weights as the B operands of the second product.  Keys outside [lo, hi] (in-page indices) are masked.
// qv: the B operand of the first product (this lane's query, chunks g, g+4, ..).
__device__ inline float score_page(const PageOperands& ops, const bf16x8 (&qv)[KSTEPS], int lo, int hi,
                                   float scale_log2, Columns& c, int g, bf16x8 (&pv)[2]) {
    f32x4 s[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < KSTEPS; ++j) acc = mfma_16x16x32(ops.k[t][j], qv[j], acc);
        s[t] = acc;
    }
    // this lane holds, for its query, keys tile_key(t, 4g + i)
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int key = tile_key(t, 4 * g + i);
            const float v = (key >= lo && key <= hi) ? s[t][i] * scale_log2 : -INFINITY;
            s[t][i] = v;
            mx = fmaxf(mx, v);
        }
    mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
    mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
    const float m_new = fmaxf(c.m, mx);
    // A column can reach a page of its tile in which it sees no key yet (a window's lower edge, a page
    // border inside a tile of queries): its maximum is still -inf then; subtracting 0 instead keeps
    // every exponential at exp2(-inf) = 0 rather than NaN.
    const float m_sub = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = exp2_weight(c.m - m_sub);       // c.m = -inf before the first visible key: 0
    float sum = 0.f;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float p = exp2_weight(s[2 * h + e / 4][e % 4] - m_sub);
            sum += p;
            pv[h][e] = (__bf16)p;
        }
    c.l = c.l * alpha + sum;                            // this lane's share; the groups are added at the end
    c.m = m_new;
    return alpha;
}

// A key beyond `hi` (an in-page index) has weight zero, but its column of V^T would still be multiplied, and pages
// are handed out uncleared: what an earlier request left there (a NaN or an infinity, if its activations overflowed)
// times zero is NaN.  So the values of such keys are taken as zero.  Only the page that holds the column's last key
// has any; this lane's fragments hold keys 32 h + 8 g + e.
__device__ inline void blank_values_after(PageOperands& ops, int hi, int g) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const bool seen = h * 32 + g * 8 + e <= hi;
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt) ops.v[dt][h][e] = seen ? ops.v[dt][h][e] : (__bf16)0.0f;
        }
}

__device__ inline void weigh_values(const PageOperands& ops, const bf16x8 (&pv)[2], float alpha, Columns& c) {
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) {
        f32x4 acc = c.o[dt] * alpha;
#pragma unroll
        for (int h = 0; h < 2; ++h) acc = mfma_16x16x32(ops.v[dt][h], pv[h], acc);
        c.o[dt] = acc;
    }
}

// All pages p0 <= p < p1 of one sequence and kv head.  The reads of the next page are issued as soon as the
// registers of the current one are free: K after the scores, V after the weighted sum, so that a page's
// latency hides behind the previous page's arithmetic.  first/last: the column's own key range.
// start.prepare(qv, c) is called once, after the first page's keys have been asked for: a caller whose query is
// not finished yet finishes it there, while the keys are on their way (Ready: nothing to do).
struct Ready {
    __device__ void prepare(bf16x8 (&)[KSTEPS], Columns&) {}
};
template <typename Start>
__device__ inline void attend_pages(const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
                                    const int* __restrict__ pages, int nkv, int kvh, int p0, int p1,
                                    bf16x8 (&qv)[KSTEPS], int first, int last, float scale_log2, Columns& c,
                                    int r, int g, Start& start) {
    if (p0 >= p1) return;
    PageOperands ops;
    size_t base = ((size_t)pages[p0] * nkv + kvh) * PAGE_TOKENS * HD;
    load_keys(k_cache + base, r, g, ops);
    start.prepare(qv, c);
    load_values(v_cache + base, r, g, ops);
    for (int p = p0; p < p1; ++p) {
        const bool more = p + 1 < p1;
        const size_t next = more ? ((size_t)pages[p + 1] * nkv + kvh) * PAGE_TOKENS * HD : base;
        bf16x8 pv[2];
        const float alpha = score_page(ops, qv, first - p * PAGE_TOKENS, last - p * PAGE_TOKENS, scale_log2, c, g, pv);
        if (more) load_keys(k_cache + next, r, g, ops);
        if (last - p * PAGE_TOKENS < PAGE_TOKENS - 1) blank_values_after(ops, last - p * PAGE_TOKENS, g);   // the same in every lane
        weigh_values(ops, pv, alpha, c);
        if (more) load_values(v_cache + next, r, g, ops);
        base = next;
    }
}

__device__ inline void load_query(const bf16_t* qrow, bool valid, int g, bf16x8 (&qv)[KSTEPS]) {
#pragma unroll
    for (int j = 0; j < KSTEPS; ++j) {
        const int chunk = j * 4 + g;
        const bool ok = valid && ((CHUNKS % 4 == 0) || chunk < CHUNKS);
        const bf16x8 v = load_bf16x8(qrow + (chunk < CHUNKS ? chunk : 0) * 8);     // qrow is always a real row
        qv[j] = ok ? v : zero_bf16x8();
    }
}

// ---- decode ---------------------------------------------------------------------------------------
// How a query at position `pos` cuts its key range into slices of whole pages.  The decode kernels and the merge
// must agree on it (the merge reads only the records of slices that hold pages), so it is written once.
struct SliceCut {
    int first;            // the first key the query sees
    int page_lo;          // the page that holds it
    int n_pages;          // pages from there to the query's own
    int per;              // pages a slice
    int live;             // slices that hold pages: 1 <= live <= n_slices
    __device__ SliceCut(int pos, int window, int n_slices) {
        first = window > 0 ? max(0, pos - window + 1) : 0;
        page_lo = first / PAGE_TOKENS;
        n_pages = pos / PAGE_TOKENS - page_lo + 1;
        per = (n_pages + n_slices - 1) / n_slices;
        live = (n_pages + per - 1) / per;
    }
    __device__ int begin(int slice) const { return page_lo + slice * per; }
    __device__ int end(int slice) const { return min(begin(slice) + per, page_lo + n_pages); }
};

// grid (slices, nkv * query groups, sequences), one wave each.  Workspace per (sequence, head, slice):
// m, l, two floats unused, then HD floats of the unnormalised output (which so start on 16 bytes).
constexpr int WORK_O = 4, WORK_STRIDE = HD + WORK_O;

// What a slice's wave leaves: with one slice the output itself, else its record in the workspace (maximum, sum, two
// floats unused, HD floats of the unnormalised output) for the merge; an empty slice leaves nothing.
__device__ inline void finish_slice(Columns& c, bool valid, int b, int head, int nh, int slice, int n_slices, bool empty,
                                    int g, float* __restrict__ work, bf16_t* __restrict__ out) {
    float l = c.l;
    l += __shfl_xor(l, 16, WAVE);
    l += __shfl_xor(l, 32, WAVE);
    if (!valid) return;
    if (n_slices == 1) {
        const float inv = 1.0f / l;
        bf16_t* o = out + ((size_t)b * nh + head) * HD;
#pragma unroll
        for (int dt = 0; dt < DTILES; ++dt) {
            uint2 four;
            four.x = (uint32_t)f32_to_bf16(c.o[dt][0] * inv).bits | ((uint32_t)f32_to_bf16(c.o[dt][1] * inv).bits << 16);
            four.y = (uint32_t)f32_to_bf16(c.o[dt][2] * inv).bits | ((uint32_t)f32_to_bf16(c.o[dt][3] * inv).bits << 16);
            *reinterpret_cast<uint2*>(o + dt * 16 + 4 * g) = four;
        }
        return;
    }
    if (empty) return;                                  // the merge does not read its record
    float* w = work + (((size_t)b * nh + head) * n_slices + slice) * WORK_STRIDE;
    if (g == 0) { w[0] = c.m; w[1] = l; }
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt)                    // the lane's four elements of a tile lie side by side: one store
        *reinterpret_cast<float4*>(w + WORK_O + dt * 16 + 4 * g) = make_float4(c.o[dt][0], c.o[dt][1], c.o[dt][2], c.o[dt][3]);
}

#if PALM_HEAD_DIM <= 128
#define DECODE_WAVES_PER_SIMD __attribute__((amdgpu_waves_per_eu(2)))     // fits without spilling up to this head size
#else
#define DECODE_WAVES_PER_SIMD
#endif
__global__ __launch_bounds__(WAVE) DECODE_WAVES_PER_SIMD void attention_decode_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_start, int nh, int nkv, float scale_log2, int window, int n_slices,
    float* __restrict__ work, bf16_t* __restrict__ out) {
    const int slice = blockIdx.x, b = blockIdx.z;
    const int G = nh / nkv, groups = (G + 15) / 16;
    const int kvh = blockIdx.y / groups, qg = blockIdx.y % groups;
    const int lane = threadIdx.x, r = lane % 16, g = lane / 16;
    const int pos = seq_start[b];                       // the query's position; keys 0..pos are in the cache
    const SliceCut cut(pos, window, n_slices);
    const int first = cut.first, p0 = cut.begin(slice), p1 = cut.end(slice);
    const int head = kvh * G + qg * 16 + r;             // this lane's query head (column r)
    const bool valid = qg * 16 + r < G;

    bf16x8 qv[KSTEPS];
    load_query(q + ((size_t)b * nh + (valid ? head : 0)) * HD, valid, g, qv);
    Columns c;
    c.m = -INFINITY;
    c.l = 0.f;
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) c.o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int* pages = block_table + (size_t)seq_slot[b] * max_pages;
    Ready ready;
    attend_pages(k_cache, v_cache, pages, nkv, kvh, p0, p1, qv, first, pos, scale_log2, c, r, g, ready);
    finish_slice(c, valid, b, head, nh, slice, n_slices, p0 >= p1, g, work, out);
}

// One wave per (sequence, head): merge the slices in a fixed order.  Lane s holds slice s's maximum and sum, the wave
// agrees on the overall maximum and on each slice's weight, then lane d sums output element d over the slices,
// AT_ONCE reads in flight at a time.  The kernel is a few KB of reads and its time is the round trips to memory
// that follow each other, so the maxima, the sums and the first round of outputs (all of them in the usual step) are
// asked for in the first instructions, before the sequence's length is known: a slice beyond those that hold pages
// of this sequence is read like the others (a launch is cut for the longest sequence a recorded step may serve; a
// shorter one's last records exist but hold what an earlier step left: one sequence of 2,048 tokens in a step
// recorded for 4,096 fills 33 of 64) and counts as nothing by a select.  (8 sequences, 12 slices: a step of 36 layers
// 4.04 ms against 4.12 with the reads where they are used.)
template <int AT_ONCE>
__global__ __launch_bounds__(WAVE) void attention_merge_kernel(const float* __restrict__ work, int n_slices, int nh,
                                                               const int* __restrict__ seq_start, int window,
                                                               bf16_t* __restrict__ out) {
    constexpr int PER = (HD + WAVE - 1) / WAVE;
    const float* w = work + (size_t)blockIdx.x * n_slices * WORK_STRIDE;
    const int lane = threadIdx.x;
    // asked for before the sequence's length is known: lane s's slice's maximum and sum, and the first round of outputs
    const float2 mine = *reinterpret_cast<const float2*>(w + (size_t)min(lane, n_slices - 1) * WORK_STRIDE);
    float v[AT_ONCE][PER];
    auto ask = [&](int s0) {
#pragma unroll
        for (int u = 0; u < AT_ONCE; ++u) {
            const float* rec = w + (size_t)min(s0 + u, n_slices - 1) * WORK_STRIDE + WORK_O;
#pragma unroll
            for (int i = 0; i < PER; ++i) v[u][i] = rec[min(lane + i * WAVE, HD - 1)];
        }
    };
    ask(0);
    const int live = SliceCut(seq_start[blockIdx.x / nh], window, n_slices).live;       // as the decode kernels cut the range
    float m = lane < live ? mine.x : -INFINITY, l = 0.f;
    for (int s = lane + WAVE; s < live; s += WAVE) m = fmaxf(m, w[(size_t)s * WORK_STRIDE]);
    m = wave_max(m);
    float wt = lane < live ? exp2_weight(mine.x - m) : 0.f;     // slice `lane`'s weight
    l = lane < live ? mine.y * wt : 0.f;
    for (int s = lane + WAVE; s < live; s += WAVE) l += w[(size_t)s * WORK_STRIDE + 1] * exp2_weight(w[(size_t)s * WORK_STRIDE] - m);
    l = wave_sum(l);
    float o[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) o[i] = 0.f;
    for (int s0 = 0; s0 < live; s0 += AT_ONCE) {
        if (s0 > 0) ask(s0);
#pragma unroll
        for (int u = 0; u < AT_ONCE; ++u) {
            const int s = s0 + u;
            float ws = 0.f;
            if (s < live) ws = s < WAVE ? __shfl(wt, s, WAVE) : exp2_weight(w[(size_t)s * WORK_STRIDE] - m);
#pragma unroll
            for (int i = 0; i < PER; ++i) o[i] += s < live ? v[u][i] * ws : 0.f;
        }
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int d = lane + i * WAVE;
        if (d < HD) out[(size_t)blockIdx.x * HD + d] = f32_to_bf16(o[i] / l);
    }
}

// slices read together by the merge: all of a step's where they are few, never more than fit in registers
static void launch_merge(hipStream_t stream, const float* work, int n_slices, int n_seqs, int nh, const int* seq_start,
                         int window, bf16_t* out) {
    if (n_slices <= 4) attention_merge_kernel<4><<<n_seqs * nh, WAVE, 0, stream>>>(work, n_slices, nh, seq_start, window, out);
    else if (n_slices <= 8) attention_merge_kernel<8><<<n_seqs * nh, WAVE, 0, stream>>>(work, n_slices, nh, seq_start, window, out);
    else attention_merge_kernel<16><<<n_seqs * nh, WAVE, 0, stream>>>(work, n_slices, nh, seq_start, window, out);
}

static int launch_attention_decode(hipStream_t stream, const void* q, const void* k_cache, const void* v_cache,
                                   const int* block_table, int max_pages, const int* seq_slot, const int* seq_start,
                                   int n_seqs, int nh, int nkv, int hd, float scale, int window, int n_slices,
                                   float* work, void* out) {
    PALM_CHECK(hd == HD, "attention_decode: this library was built for head size %d, not %d", HD, hd);
    PALM_CHECK(n_seqs >= 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attention_decode: seqs=%d heads=%d kv=%d", n_seqs, nh, nkv);
    PALM_CHECK(n_slices >= 1 && n_slices <= 65535, "attention_decode: %d slices", n_slices);
    PALM_CHECK(n_slices == 1 || work, "attention_decode: more than one slice needs a workspace");
    PALM_CHECK(window >= 0 && max_pages > 0, "attention_decode: window=%d max_pages=%d", window, max_pages);
    if (n_seqs == 0) return 0;
    const int groups = (nh / nkv + 15) / 16;
    PALM_CHECK(nkv * groups <= 65535 && n_seqs <= 65535, "attention_decode: grid too large");
    dim3 grid(n_slices, nkv * groups, n_seqs);
    attention_decode_kernel<<<grid, WAVE, 0, stream>>>((const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache,
                                                      block_table, max_pages, seq_slot, seq_start, nh, nkv, scale * LOG2E,
                                                      window, n_slices, work, (bf16_t*)out);
    PALM_LAUNCHED();
    if (n_slices > 1) {
        launch_merge(stream, work, n_slices, n_seqs, nh, seq_start, window, (bf16_t*)out);
        PALM_LAUNCHED();
    }
    return 0;
}

PALM_API int palm_attention_decode(hipStream_t stream, const void* q, const void* k_cache, const void* v_cache,
                                   const int* block_table, int max_pages, const int* seq_slot, const int* seq_start,
                                   int n_seqs, int nh, int nkv, int hd, float scale, int window, int n_slices,
                                   float* work, void* out) {
    return launch_attention_decode(stream, q, k_cache, v_cache, block_table, max_pages, seq_slot, seq_start, n_seqs, nh, nkv,
                                   hd, scale, window, n_slices, work, out);
}

// ---- decode with the q/k/v pass folded in -----------------------------------------------------------
// The same grid and the same slices, but the kernel starts from the joined projection's output (whole rows, or
// float32 planes of partial sums to be added) instead of a finished query: every wave adds the planes of its query
// heads, norms and rotates them (the arithmetic of qk_norm_rope_store_kernel, with a lane holding chunks g, g + 4, ..
// of its head, so that a rotation pair (i, i + HD/2) lies in one lane).  The cache does not hold the new position's
// key and value yet: the slice whose pages include that position makes them too, writes them to the cache for the
// steps to come, and starts its softmax state from them (one key: weight 1, the output the value itself); the pages
// are then walked up to the position before.  A step saves a launch and the finished query's way through memory.
// Served: head sizes that are multiples of 64 (the pair in one lane), and a rotation that is half-split over the
// whole head, or none.
constexpr bool FUSED_SERVES_HEAD = HD % 64 == 0;
constexpr int LANE_ELEMS = (HD + WAVE - 1) / WAVE;          // elements d = lane + 64 i of a head that a lane holds
constexpr int LANE_PAIRS = (HD / 2 + WAVE - 1) / WAVE;      // rotation pairs (i, i + HD/2), i = lane + 64 ii

// Eight consecutive elements as they come from memory; widened only where they are used, so that a read can be
// asked for long before.
template <typename TIN> struct Raw8;
template <> struct Raw8<float> {
    float4 a, b;
    __device__ void read(const float* p) { a = *reinterpret_cast<const float4*>(p); b = *reinterpret_cast<const float4*>(p + 4); }
    __device__ void widen(float (&x)[8]) const { x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w; x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w; }
};
template <> struct Raw8<bf16_t> {
    uint4 u;
    __device__ void read(const bf16_t* p) { u = *reinterpret_cast<const uint4*>(p); }
    __device__ void widen(float (&x)[8]) const {
        x[0] = __uint_as_float(u.x << 16); x[1] = __uint_as_float(u.x & 0xffff0000u);
        x[2] = __uint_as_float(u.y << 16); x[3] = __uint_as_float(u.y & 0xffff0000u);
        x[4] = __uint_as_float(u.z << 16); x[5] = __uint_as_float(u.z & 0xffff0000u);
        x[6] = __uint_as_float(u.w << 16); x[7] = __uint_as_float(u.w & 0xffff0000u);
    }
};

// The step's rows and what is to be done with them.  ask() only asks memory for what does not depend on the
// sequence's length (the rows, the norm weights, the rotation), so that it can stand at the kernel's very start and
// the answers arrive while the page table is being looked up; prepare() does the arithmetic.
template <typename TIN, int PLANES>
struct FromProjection {
    static constexpr int HELD = PLANES > 0 ? PLANES : 1;          // planes whose reads are on their way together
    const TIN* q_row;  const TIN* k_row;  const TIN* v_row;      // this lane's query head, the kv head's key and value
    int planes;  size_t plane_stride;
    const float* q_norm_w;  const float* k_norm_w;  float eps;
    const float* cos_row;  const float* sin_row;
    float scale_log2;
    bool valid;          // the lane's column is a query head
    bool owner;          // this wave's slice holds the new position's page, and the layer writes its cache
    bf16_t* k_dst;  bf16_t* v_dst;                               // where the new key's row and the new value's column start
    int r, g, lane;
    float* k_vals;  float* v_vals;                               // HD floats each in LDS
    // asked for at the start
    Raw8<TIN> q_raw[HELD][KSTEPS];
    Raw8<float> qw_raw[KSTEPS], cos_raw[KSTEPS / 2 > 0 ? KSTEPS / 2 : 1], sin_raw[KSTEPS / 2 > 0 ? KSTEPS / 2 : 1];
    TIN k_raw[HELD][LANE_ELEMS], v_raw[HELD][LANE_ELEMS];
    float kw_raw[LANE_ELEMS], k_cos[LANE_PAIRS], k_sin[LANE_PAIRS];

    __device__ void ask() {
#pragma unroll
        for (int pl = 0; pl < HELD; ++pl)
#pragma unroll
            for (int j = 0; j < KSTEPS; ++j) q_raw[pl][j].read(q_row + pl * plane_stride + (j * 4 + g) * 8);
        if (q_norm_w) {
#pragma unroll
            for (int j = 0; j < KSTEPS; ++j) qw_raw[j].read(q_norm_w + (j * 4 + g) * 8);
        }
        if (cos_row) {
#pragma unroll
            for (int j = 0; j < KSTEPS / 2; ++j) {
                cos_raw[j].read(cos_row + (j * 4 + g) * 8);
                sin_raw[j].read(sin_row + (j * 4 + g) * 8);
            }
        }
        // the new key and value, spread over the wave; every slice asks (a few bytes), the owner uses them
#pragma unroll
        for (int i = 0; i < LANE_ELEMS; ++i) {
            const int d = lane + WAVE * i;
#pragma unroll
            for (int pl = 0; pl < HELD; ++pl) {
                k_raw[pl][i] = k_row[pl * plane_stride + d];
                v_raw[pl][i] = v_row[pl * plane_stride + d];
            }
            kw_raw[i] = k_norm_w ? k_norm_w[d] : 1.f;
        }
#pragma unroll
        for (int ii = 0; ii < LANE_PAIRS; ++ii) {
            const int i = min(lane + WAVE * ii, HD / 2 - 1);
            k_cos[ii] = cos_row ? cos_row[i] : 1.f;
            k_sin[ii] = cos_row ? sin_row[i] : 0.f;
        }
    }

    __device__ void prepare(bf16x8 (&qv)[KSTEPS], Columns& c) {
        // the query: planes added in their order, RMS norm over the head (the four lanes of a column share a head),
        // rotation of (i, i + HD/2), rounding
        float x[KSTEPS][8];
#pragma unroll
        for (int j = 0; j < KSTEPS; ++j) {
            q_raw[0][j].widen(x[j]);
#pragma unroll
            for (int pl = 1; pl < HELD; ++pl) {
                float y[8];
                q_raw[pl][j].widen(y);
#pragma unroll
                for (int e = 0; e < 8; ++e) x[j][e] += y[e];
            }
        }
        if (PLANES == 0) {
            for (int pl = 1; pl < planes; ++pl) {
#pragma unroll
                for (int j = 0; j < KSTEPS; ++j) {
                    Raw8<TIN> more;
                    float y[8];
                    more.read(q_row + pl * plane_stride + (j * 4 + g) * 8);
                    more.widen(y);
#pragma unroll
                    for (int e = 0; e < 8; ++e) x[j][e] += y[e];
                }
            }
        }
        if (q_norm_w) {
            float ss = 0.f;
#pragma unroll
            for (int j = 0; j < KSTEPS; ++j)
#pragma unroll
                for (int e = 0; e < 8; ++e) ss += x[j][e] * x[j][e];
            ss += __shfl_xor(ss, 16, WAVE);
            ss += __shfl_xor(ss, 32, WAVE);
            const float inv = 1.0f / sqrtf(ss / (float)HD + eps);
#pragma unroll
            for (int j = 0; j < KSTEPS; ++j) {
                float w[8];
                qw_raw[j].widen(w);
#pragma unroll
                for (int e = 0; e < 8; ++e) x[j][e] = x[j][e] * inv * w[e];
            }
        }
        if (cos_row) {
#pragma unroll
            for (int j = 0; j < KSTEPS / 2; ++j) {
                float cs[8], sn[8];
                cos_raw[j].widen(cs);
                sin_raw[j].widen(sn);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float x0 = x[j][e], x1 = x[j + KSTEPS / 2][e];
                    x[j][e] = x0 * cs[e] - x1 * sn[e];
                    x[j + KSTEPS / 2][e] = x0 * sn[e] + x1 * cs[e];
                }
            }
        }
#pragma unroll
        for (int j = 0; j < KSTEPS; ++j)
#pragma unroll
            for (int e = 0; e < 8; ++e) qv[j][e] = valid ? (__bf16)x[j][e] : (__bf16)0.f;
        if (!owner) return;

        // the new key and value, element d = lane + 64 i in this lane, as qk_norm_rope_store_kernel makes them
        float kx[LANE_ELEMS], vx[LANE_ELEMS], ss = 0.f;
#pragma unroll
        for (int i = 0; i < LANE_ELEMS; ++i) {
            kx[i] = to_float(k_raw[0][i]);
            vx[i] = to_float(v_raw[0][i]);
#pragma unroll
            for (int pl = 1; pl < HELD; ++pl) {
                kx[i] += to_float(k_raw[pl][i]);
                vx[i] += to_float(v_raw[pl][i]);
            }
            if (PLANES == 0) {
                for (int pl = 1; pl < planes; ++pl) {
                    kx[i] += to_float(k_row[pl * plane_stride + lane + WAVE * i]);
                    vx[i] += to_float(v_row[pl * plane_stride + lane + WAVE * i]);
                }
            }
            ss += kx[i] * kx[i];
        }
        if (k_norm_w) {
            ss = wave_sum(ss);
            const float inv = 1.0f / sqrtf(ss / (float)HD + eps);
#pragma unroll
            for (int i = 0; i < LANE_ELEMS; ++i) kx[i] = kx[i] * inv * kw_raw[i];
        }
#pragma unroll
        for (int i = 0; i < LANE_ELEMS; ++i) {
            const int d = lane + WAVE * i;
            const bf16_t v_rounded = f32_to_bf16(vx[i]);
            k_vals[d] = kx[i];
            v_vals[d] = to_float(v_rounded);
            v_dst[(size_t)d * PAGE_TOKENS] = v_rounded;
        }
        __syncthreads();                                 // the block is this one wave
        if (cos_row) {
#pragma unroll
            for (int ii = 0; ii < LANE_PAIRS; ++ii) {
                const int i = lane + WAVE * ii;
                if (i < HD / 2) {
                    const float x0 = k_vals[i], x1 = k_vals[i + HD / 2];
                    k_vals[i] = x0 * k_cos[ii] - x1 * k_sin[ii];
                    k_vals[i + HD / 2] = x0 * k_sin[ii] + x1 * k_cos[ii];
                }
            }
            __syncthreads();
        }
        // its score against the finished query, both as the cache and the matrix cores hold them
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < KSTEPS; ++j) {
            Raw8<float> chunk;
            float kf[8];
            bf16x8 kb;
            chunk.read(k_vals + (j * 4 + g) * 8);
            chunk.widen(kf);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                kb[e] = (__bf16)kf[e];
                s += (float)qv[j][e] * (float)kb[e];
            }
            if (r == 0) *reinterpret_cast<bf16x8*>(k_dst + (j * 4 + g) * 8) = kb;      // lanes (0, g): the whole row
        }
        s += __shfl_xor(s, 16, WAVE);
        s += __shfl_xor(s, 32, WAVE);
        // one key: its weight is exp2(s - s) = 1; the sum's share lies with group 0, the others hold none
        c.m = s * scale_log2;
        c.l = g == 0 ? 1.f : 0.f;
#pragma unroll
        for (int dt = 0; dt < DTILES; ++dt) {           // this lane's output elements 16 dt + 4 g .. + 3
            const float4 four = *reinterpret_cast<const float4*>(v_vals + dt * 16 + 4 * g);
            c.o[dt] = f32x4{four.x, four.y, four.z, four.w};
        }
    }
};

template <typename TIN, int PLANES>
__global__ __launch_bounds__(WAVE) DECODE_WAVES_PER_SIMD void attention_decode_fused_kernel(
    const TIN* __restrict__ qkv, int planes, size_t plane_stride, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, float eps, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    int write_cache, bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_start, int nh, int nkv, float scale_log2, int window, int n_slices,
    float* __restrict__ work, bf16_t* __restrict__ out) {
    if constexpr (FUSED_SERVES_HEAD) {
        __shared__ float new_key[HD], new_value[HD];
        const int slice = blockIdx.x, b = blockIdx.z;
        const int G = nh / nkv, groups = (G + 15) / 16;
        const int kvh = blockIdx.y / groups, qg = blockIdx.y % groups;
        const int lane = threadIdx.x, r = lane % 16, g = lane / 16;
        const int head = kvh * G + qg * 16 + r;
        const bool valid = qg * 16 + r < G;

        FromProjection<TIN, PLANES> start;
        const TIN* row = qkv + (size_t)b * (nh + 2 * nkv) * HD;
        start.q_row = row + (size_t)(valid ? head : 0) * HD;
        start.k_row = row + (size_t)(nh + kvh) * HD;
        start.v_row = row + (size_t)(nh + nkv + kvh) * HD;
        start.planes = planes;
        start.plane_stride = plane_stride;
        start.q_norm_w = q_norm_w;
        start.k_norm_w = k_norm_w;
        start.eps = eps;
        start.cos_row = cos_t ? cos_t + (size_t)b * (HD / 2) : nullptr;
        start.sin_row = sin_t ? sin_t + (size_t)b * (HD / 2) : nullptr;
        start.scale_log2 = scale_log2;
        start.valid = valid;
        start.r = r;
        start.g = g;
        start.lane = lane;
        start.k_vals = new_key;
        start.v_vals = new_value;
        start.ask();

        const int pos = seq_start[b];
        const SliceCut cut(pos, window, n_slices);
        const int first = cut.first, p0 = cut.begin(slice), p1 = cut.end(slice);
        const int* pages = block_table + (size_t)seq_slot[b] * max_pages;
        const int page = pos / PAGE_TOKENS;
        start.owner = write_cache && page >= p0 && page < p1;
        start.k_dst = start.v_dst = nullptr;
        if (start.owner) {
            const size_t at = ((size_t)pages[page] * nkv + kvh) * PAGE_TOKENS * HD;
            start.k_dst = k_cache + at + (size_t)(pos % PAGE_TOKENS) * HD;
            start.v_dst = v_cache + at + pos % PAGE_TOKENS;
        }

        bf16x8 qv[KSTEPS];
        Columns c;
        c.m = -INFINITY;
        c.l = 0.f;
#pragma unroll
        for (int dt = 0; dt < DTILES; ++dt) c.o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
        // with a key and value of its own making the step sees the cache up to the position before
        attend_pages(k_cache, v_cache, pages, nkv, kvh, p0, p1, qv, first, write_cache ? pos - 1 : pos, scale_log2, c, r, g, start);
        finish_slice(c, valid, b, head, nh, slice, n_slices, p0 >= p1, g, work, out);
    }
}

PALM_API int palm_attention_decode_fused_serves(int rotary_dim, int pairing) {
    return FUSED_SERVES_HEAD && (rotary_dim == 0 || (rotary_dim == HD && pairing == 0));
}

// qkv: [n_seqs, (nh + 2 nkv) hd] bfloat16 (qkv_is_planes = 0), or [planes, n_seqs, (nh + 2 nkv) hd] float32.
// cos_t, sin_t: [n_seqs, hd / 2] float32 rows of the sequences' positions, or both null for no rotation.
// Without write_cache the cache already holds the new position's key and value (a layer that reads another's).
PALM_API int palm_attention_decode_fused(hipStream_t stream, const void* qkv, int qkv_is_planes, int planes,
                                         const float* q_norm_w, const float* k_norm_w, float eps, const float* cos_t,
                                         const float* sin_t, int rotary_dim, int pairing, int write_cache, void* k_cache,
                                         void* v_cache, const int* block_table, int max_pages, const int* seq_slot,
                                         const int* seq_start, int n_seqs, int nh, int nkv, int hd, float scale,
                                         int window, int n_slices, float* work, void* out) {
    PALM_CHECK(hd == HD, "attention_decode_fused: this library was built for head size %d, not %d", HD, hd);
    PALM_CHECK((cos_t == nullptr) == (sin_t == nullptr), "attention_decode_fused: cos and sin tables come together");
    PALM_CHECK(palm_attention_decode_fused_serves(cos_t ? rotary_dim : 0, pairing),
               "attention_decode_fused: head size %d with rotation over %d (pairing %d) is not served: the head size must be a "
               "multiple of 64 and the rotation half-split over the whole head, or absent", HD, rotary_dim, pairing);
    PALM_CHECK((q_norm_w == nullptr) == (k_norm_w == nullptr), "attention_decode_fused: q and k norm weights come together");
    PALM_CHECK(n_seqs >= 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attention_decode_fused: seqs=%d heads=%d kv=%d", n_seqs, nh, nkv);
    PALM_CHECK(n_slices >= 1 && n_slices <= 65535, "attention_decode_fused: %d slices", n_slices);
    PALM_CHECK(n_slices == 1 || work, "attention_decode_fused: more than one slice needs a workspace");
    PALM_CHECK(window >= 0 && max_pages > 0, "attention_decode_fused: window=%d max_pages=%d", window, max_pages);
    PALM_CHECK(planes >= 1 && (qkv_is_planes || planes == 1), "attention_decode_fused: %d planes of whole rows", planes);
    if (n_seqs == 0) return 0;
    const int groups = (nh / nkv + 15) / 16;
    PALM_CHECK(nkv * groups <= 65535 && n_seqs <= 65535, "attention_decode_fused: grid too large");
    dim3 grid(n_slices, nkv * groups, n_seqs);
    const size_t plane_stride = (size_t)n_seqs * (nh + 2 * nkv) * HD;
#define PALM_FUSED(TIN, P) attention_decode_fused_kernel<TIN, P><<<grid, WAVE, 0, stream>>>( \
        (const TIN*)qkv, planes, plane_stride, q_norm_w, k_norm_w, eps, cos_t, sin_t, write_cache, (bf16_t*)k_cache, \
        (bf16_t*)v_cache, block_table, max_pages, seq_slot, seq_start, nh, nkv, scale * LOG2E, window, n_slices, work, (bf16_t*)out)
    if (!qkv_is_planes) PALM_FUSED(bf16_t, 1);
    else if (planes == 1) PALM_FUSED(float, 1);
    else if (planes == 2) PALM_FUSED(float, 2);
    else PALM_FUSED(float, 0);
#undef PALM_FUSED
    PALM_LAUNCHED();
    if (n_slices > 1) {
        launch_merge(stream, work, n_slices, n_seqs, nh, seq_start, window, (bf16_t*)out);
        PALM_LAUNCHED();
    }
    return 0;
}

// ---- decode without a workspace argument ------------------------------------------------------------
// The slices' partial results go through this array instead of a buffer of the caller's.  Each GPU has a copy of
// its own at an address of its own; in host code the array's name is only a handle for hipGetSymbolAddress, never
// a pointer to hand to a kernel.  The address is asked for once per device, with that device current, and kept.
constexpr long long STATIC_WORK_FLOATS = 2ll * 1024 * 1024;            // 8 MiB
static __device__ __align__(256) float scratch[STATIC_WORK_FLOATS];
constexpr int STATIC_MAX_DEVICES = 64;
static float* g_scratch_of_device[STATIC_MAX_DEVICES];                  // null until the device's first call
static std::mutex g_scratch_lock;

PALM_API long long palm_attention_decode_static_limit() { return STATIC_WORK_FLOATS; }

// The current device's copy of the array (null and an error text on failure).
static float* scratch_of_current_device() {
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) { palm_fail("attention_decode_static: hipGetDevice failed: %s", hipGetErrorString(e)); return nullptr; }
    if (device < 0 || device >= STATIC_MAX_DEVICES) {
        palm_fail("attention_decode_static: device %d is beyond the %d this library keeps a buffer for", device, STATIC_MAX_DEVICES);
        return nullptr;
    }
    std::lock_guard<std::mutex> hold(g_scratch_lock);
    if (!g_scratch_of_device[device]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            palm_fail("attention_decode_static: hipGetSymbolAddress failed on device %d: %s", device, hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_of_device[device] = static_cast<float*>(ptr);
    }
    return g_scratch_of_device[device];
}

PALM_API int palm_attention_decode_static(hipStream_t stream, const void* q, const void* k_cache, const void* v_cache,
                                          const int* block_table, int max_pages, const int* seq_slot,
                                          const int* seq_start, int n_seqs, int nh, int nkv, int hd, float scale,
                                          int window, int n_slices, void* out) {
    PALM_CHECK(n_seqs >= 0 && nh > 0 && n_slices >= 1, "attention_decode_static: seqs=%d heads=%d slices=%d", n_seqs, nh, n_slices);
    const long long need = n_slices > 1 ? (long long)n_seqs * nh * n_slices * WORK_STRIDE : 0;
    PALM_CHECK(need <= STATIC_WORK_FLOATS,
               "attention_decode_static: %d sequences x %d heads x %d slices x %d floats = %lld floats exceed the library's "
               "buffer of %lld; use fewer slices, or palm_attention_decode with a workspace of the caller's",
               n_seqs, nh, n_slices, WORK_STRIDE, need, STATIC_WORK_FLOATS);
    float* work = nullptr;
    if (n_slices > 1) {
        work = scratch_of_current_device();
        if (!work) return -1;
    }
    return launch_attention_decode(stream, q, k_cache, v_cache, block_table, max_pages, seq_slot, seq_start, n_seqs, nh, nkv,
                                   hd, scale, window, n_slices, work, out);
}

// ---- prefill --------------------------------------------------------------------------------------
// A block of four waves serves one kv head, up to eight query heads of its group (more heads: more blocks)
// and a tile of QB query positions, QB = 16 * max(1, 8 / heads): at most eight "units" (two a wave) of 16 columns
// (head, 16 positions), two for each wave.  A page of K and of V^T is read from memory once for the block,
// into LDS; every wave takes its MFMA operands from there, each operand serving both of its units.  The next
// page is on its way into registers while the current one is being used.
// Causal attention gives a late tile of queries many more keys than an early one, and all blocks of a launch
// run at once, so blocks of unequal work would leave half the chip waiting for the last ones.  A block's
// 16-query sub-tiles are therefore taken alternately from the front and from the back of the sequence's new
// tokens (sub-tile f with sub-tile N - 1 - f): every block then has about the same number of (unit, page)
// products.  The early sub-tile's keys are among the late one's, so the block walks the late one's pages and
// the early one's units just stop taking part (`active`) once the pages lie beyond them.
// (Eight waves a block, 16 units, halve what a block's queries read of K and V from L2; measured at 2,048 tokens:
// 77 us against 64, the barrier of eight waves and one block a compute unit costing more than the reads save.)
#ifndef PALM_PF_WAVES
#define PALM_PF_WAVES 4
#endif
constexpr int PF_WAVES = PALM_PF_WAVES;
constexpr int PF_THREADS = PF_WAVES * WAVE;
constexpr int PF_UNITS = 2;                                // units of 16 columns held by a wave
constexpr float PF_LAZY_LOG2 = 8.0f;                       // how far (in powers of two) a maximum may rise before the outputs are rescaled
// K rows in LDS are a multiple of eight 16-byte chunks long and a row's chunks are permuted by its number
// (chunk ^ swizzle(row)): the eight lanes that LDS serves together read one chunk column of keys
// {0..3, 8..11} (or {4..7, 12..15}, ..), which the permutation sends to eight different bank groups.
constexpr int K_CHUNKS = (CHUNKS + 7) / 8 * 8;
constexpr int K_STRIDE = K_CHUNKS * 8;
__device__ inline int k_swizzle(int row) { return (row & 3) | (((row >> 3) & 1) << 2); }
// Head sizes whose key rows are whole multiples of 128 bytes and of which a whole number fills 1 KB (64, 128)
// take their pages from memory straight into LDS (global_load_lds: no registers in between, no write
// instruction); a wave's instruction fills 1 KB of LDS in lane order, so rows cannot be padded there and V^T's
// chunks are permuted like K's instead (row d's chunk c at c ^ v_swizzle(d): the 16 rows that lanes read together
// then start in 16 different groups of four banks).  A row of 192 elements (24 chunks) would straddle two
// instructions' kilobytes, which page_sources() does not describe: such sizes go through registers.
constexpr bool PF_DMA = CHUNKS % 8 == 0 && WAVE % CHUNKS == 0 && (PAGE_TOKENS * K_STRIDE + HD * PAGE_TOKENS) * 2 <= 60 * 1024;
constexpr int V_STRIDE = PF_DMA ? PAGE_TOKENS : PAGE_TOKENS + 8;
__device__ inline int v_swizzle(int row) { return PF_DMA ? (row >> 1) & 7 : 0; }
constexpr int PAGE_CHUNKS = PAGE_TOKENS * HD / 8;          // 16-byte chunks in a page of K (and of V^T)
constexpr int PF_LOADS = (PAGE_CHUNKS + PF_THREADS - 1) / PF_THREADS;
constexpr bool PF_SHARE = (PAGE_TOKENS * K_STRIDE + HD * V_STRIDE) * 2 > 60 * 1024;   // too big for 64 KB: V reuses K's space

struct PagePrefetch { bf16x8 k[PF_LOADS], v[PF_LOADS]; };

__device__ inline void prefetch_keys(const bf16_t* __restrict__ kp, PagePrefetch& pf) {
#pragma unroll
    for (int i = 0; i < PF_LOADS; ++i) {
        const int c = i * PF_THREADS + threadIdx.x;
        pf.k[i] = load_bf16x8(kp + (size_t)(c < PAGE_CHUNKS ? c : 0) * 8);
    }
}
__device__ inline void prefetch_values(const bf16_t* __restrict__ vp, PagePrefetch& pf) {
#pragma unroll
    for (int i = 0; i < PF_LOADS; ++i) {
        const int c = i * PF_THREADS + threadIdx.x;
        pf.v[i] = load_bf16x8(vp + (size_t)(c < PAGE_CHUNKS ? c : 0) * 8);
    }
}
__device__ inline void stage_keys(const PagePrefetch& pf, bf16_t* k_lds) {
#pragma unroll
    for (int i = 0; i < PF_LOADS; ++i) {
        const int c = i * PF_THREADS + threadIdx.x;
        if (c < PAGE_CHUNKS) *reinterpret_cast<bf16x8*>(k_lds + (c / CHUNKS) * K_STRIDE + ((c % CHUNKS) ^ k_swizzle(c / CHUNKS)) * 8) = pf.k[i];
    }
}
__device__ inline void stage_values(const PagePrefetch& pf, bf16_t* v_lds) {
#pragma unroll
    for (int i = 0; i < PF_LOADS; ++i) {
        const int c = i * PF_THREADS + threadIdx.x;
        if (c < PAGE_CHUNKS) *reinterpret_cast<bf16x8*>(v_lds + (c / 8) * V_STRIDE + ((c % 8) ^ v_swizzle(c / 8)) * 8) = pf.v[i];
    }
}

// A page of K and of V^T from memory into LDS without a stop in registers.  An instruction of a wave fills 1 KB
// in lane order: for K that is 64 / CHUNKS key rows, for V^T eight rows of 64 tokens; a lane asks for the chunk
// that belongs at its place.  k_from / v_from: the lane's places in a page, as page_sources() gives them.
struct PageSources { uint32_t k[PF_LOADS], v[PF_LOADS]; };       // byte offsets into a page of K and of V^T
__device__ inline PageSources page_sources() {
    PageSources src;
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    static_assert(!PF_DMA || WAVE % CHUNKS == 0, "an instruction's 64 chunks must be whole key rows");
    constexpr int K_ROWS = WAVE / CHUNKS;                        // key rows an instruction covers
#pragma unroll
    for (int i = 0; i < PF_LOADS; ++i) {
        const int inst = i * PF_WAVES + wave;
        const int k_row = inst * K_ROWS + lane / CHUNKS, v_row = inst * 8 + lane / 8;
        src.k[i] = (uint32_t)(k_row * HD + ((lane % CHUNKS) ^ k_swizzle(k_row)) * 8) * sizeof(bf16_t);
        src.v[i] = (uint32_t)(v_row * PAGE_TOKENS + ((lane % 8) ^ v_swizzle(v_row)) * 8) * sizeof(bf16_t);
    }
    return src;
}
// The load itself is written out in assembly.  Through the compiler's builtin every later read of LDS, of either
// buffer, would first wait for all such loads, and the page on its way would never overlap the arithmetic on the
// page at hand.  This way the compiler does not know of the loads: lds_loads_done() waits for them before the
// barrier after which their buffer is read (a wait of the compiler's own for other loads can only wait for these
// too, since loads come back in order).
__device__ __forceinline__ void load_16_bytes_a_lane_into_lds(const void* from, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(from), "s"(lds_base) : "m0");
}
// s_waitcnt vmcnt(0), as an instruction that the compiler knows (it then also knows that its own loads are done)
__device__ __forceinline__ void lds_loads_done() { __builtin_amdgcn_s_waitcnt(0x0F70); }
__device__ __forceinline__ uint32_t lds_address(const bf16_t* p) {       // the same in every lane of a wave
    return __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p);
}
__device__ inline void page_into_lds(const bf16_t* __restrict__ kp, const bf16_t* __restrict__ vp, const PageSources& src,
                                     bf16_t* k_lds, bf16_t* v_lds) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    constexpr int KB = 1024 / sizeof(bf16_t);                    // elements of 1 KB
#pragma unroll
    for (int i = 0; i < PF_LOADS; ++i)
        load_16_bytes_a_lane_into_lds(reinterpret_cast<const char*>(kp) + src.k[i], lds_address(k_lds + (i * PF_WAVES + wave) * KB));
#pragma unroll
    for (int i = 0; i < PF_LOADS; ++i)
        load_16_bytes_a_lane_into_lds(reinterpret_cast<const char*>(vp) + src.v[i], lds_address(v_lds + (i * PF_WAVES + wave) * KB));
}

// The page that holds a sequence's last key also holds, beyond it, what an earlier owner of the page left there
// (pages are handed out uncleared).  Those keys have weight zero in every column, but their columns of V^T are
// multiplied all the same, and zero times a NaN or an infinity is NaN: they are made zero in LDS, once, before the
// page is used.  `tail`: the last key of the sequence, as an index into the page.  (A barrier must follow.)
__device__ inline void blank_values_after(bf16_t* v_lds, int tail) {
    for (int idx = threadIdx.x; idx < HD * (PAGE_TOKENS / 8); idx += PF_THREADS) {
        const int d = idx / (PAGE_TOKENS / 8), chunk = idx % (PAGE_TOKENS / 8);
        if (chunk * 8 + 7 <= tail) continue;
        bf16x8* at = reinterpret_cast<bf16x8*>(v_lds + d * V_STRIDE + (chunk ^ v_swizzle(d)) * 8);
        bf16x8 v = *at;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = chunk * 8 + e <= tail ? v[e] : (__bf16)0.0f;
        *at = v;
    }
}

struct Unit {                 // one (head, 16 query positions): the wave's share of it
    bool live;                // false: the wave has no such unit (fewer units than slots)
    bool active;              // the page at hand holds keys that some column of the unit sees
    int page_lo, page_hi;     // the pages that do
    bool valid;               // this lane's column is a real query
    int pos, first;           // the column's position and the first key it sees
    size_t row;               // the column's row in q and out
    int head;
    bf16x8 qv[KSTEPS];
    Columns c;                // (c.l is not used here: see weights)
    f32x4 weights;            // the sum of the column's softmax weights, four times
};

__device__ inline void read_key_fragments(const bf16_t* k_lds, int t, int r, int g, bf16x8 (&kf)[KSTEPS]) {
    const int key_row = tile_key(t, r);
    const bf16_t* krow = k_lds + key_row * K_STRIDE;
#pragma unroll
    for (int j = 0; j < KSTEPS; ++j) {
        const int chunk = j * 4 + g;
        const bool ok = (CHUNKS % 4 == 0) || chunk < CHUNKS;
        kf[j] = *reinterpret_cast<const bf16x8*>(krow + ((ok ? chunk : 0) ^ k_swizzle(key_row)) * 8);
        if (!ok) kf[j] = zero_bf16x8();
    }
}

// Scores and softmax of one page for the wave's units.  The fragments of key tile t+1 are read from LDS
// before the products of tile t run, so a read's latency hides behind arithmetic.  `interior`: every key of
// the page is visible to every column of the wave (the usual case away from the diagonal), no masking then.
__device__ inline void unit_scores(const bf16_t* k_lds, Unit (&u)[PF_UNITS], int page_first_key, float scale_log2,
                                   int r, int g, bool interior, bf16x8 (&pv)[PF_UNITS][2], float (&alpha)[PF_UNITS]) {
    f32x4 s[PF_UNITS][4];
    bf16x8 kf[2][KSTEPS];
    read_key_fragments(k_lds, 0, r, g, kf[0]);
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        if (t < 3) read_key_fragments(k_lds, t + 1, r, g, kf[(t + 1) & 1]);
#pragma unroll
        for (int x = 0; x < PF_UNITS; ++x) {
            if (!u[x].active) continue;                         // (its scores stay unset and unused)
            f32x4 acc = mfma_16x16x32(kf[t & 1][0], u[x].qv[0], f32x4{0.f, 0.f, 0.f, 0.f});
#pragma unroll
            for (int j = 1; j < KSTEPS; ++j) acc = mfma_16x16x32(kf[t & 1][j], u[x].qv[j], acc);
            s[x][t] = acc;
        }
    }
#pragma unroll
    for (int x = 0; x < PF_UNITS; ++x) {
        Columns& c = u[x].c;
        alpha[x] = 1.0f;
        if (!u[x].active) continue;
        float mx = -INFINITY;
        if (interior) {
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) mx = fmaxf(mx, s[x][t][i]);
        } else {
            const int lo = u[x].first - page_first_key, hi = u[x].pos - page_first_key;
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int key = tile_key(t, 4 * g + i);
                    const float v = (key >= lo && key <= hi) ? s[x][t][i] : -INFINITY;
                    s[x][t][i] = v;
                    mx = fmaxf(mx, v);
                }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
        mx *= scale_log2;                                           // the scale is positive: the maximum commutes with it
        // c.m is the reference the weights are taken against, not the running maximum itself: it follows the
        // maximum only when that has risen by more than PF_LAZY_LOG2 above it (from -inf: at the first key).
        // Until then the weights are at most 2^PF_LAZY_LOG2 instead of at most 1, which 32-bit sums and the
        // bfloat16 operand hold as well, and the outputs need no rescaling.
        const bool jump = mx > c.m + PF_LAZY_LOG2;
        const float m_ref = jump ? mx : c.m;
        const float m_sub = m_ref == -INFINITY ? 0.f : m_ref;       // see score_page
        alpha[x] = jump ? exp2_weight(c.m - m_sub) : 1.0f;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int e = 0; e < 8; ++e)
                pv[x][h][e] = (__bf16)exp2_weight(fmaf(s[x][2 * h + e / 4][e % 4], scale_log2, -m_sub));
        c.m = m_ref;
    }
}

// The weighted values of one page.  `rescale` false: no column's maximum moved (every alpha is 1), the
// outputs stay where the matrix cores keep them.
__device__ inline void unit_values(const bf16_t* v_lds, Unit (&u)[PF_UNITS], int r, int g,
                                   const bf16x8 (&pv)[PF_UNITS][2], const float (&alpha)[PF_UNITS], bool rescale) {
    if (rescale) {
#pragma unroll
        for (int x = 0; x < PF_UNITS; ++x) {
            if (!u[x].active) continue;
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt) u[x].c.o[dt] = u[x].c.o[dt] * alpha[x];
            u[x].weights = u[x].weights * alpha[x];
        }
    }
    // the sum of a column's weights comes from the matrix cores too: a row of ones in place of a row of V^T (every
    // row of the tile is that row: each of a lane's four elements is the whole sum over the page's keys)
    bf16x8 ones;
#pragma unroll
    for (int e = 0; e < 8; ++e) ones[e] = (__bf16)1.0f;
#pragma unroll
    for (int x = 0; x < PF_UNITS; ++x) {
        if (!u[x].active) continue;
#pragma unroll
        for (int h = 0; h < 2; ++h) u[x].weights = mfma_16x16x32(ones, pv[x][h], u[x].weights);
    }
    bf16x8 vf[2][2];
#pragma unroll
    for (int h = 0; h < 2; ++h) vf[0][h] = *reinterpret_cast<const bf16x8*>(v_lds + r * V_STRIDE + ((h * 4 + g) ^ v_swizzle(r)) * 8);
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) {
        if (dt + 1 < DTILES) {
            const bf16_t* vrow = v_lds + ((dt + 1) * 16 + r) * V_STRIDE;
#pragma unroll
            for (int h = 0; h < 2; ++h)
                vf[(dt + 1) & 1][h] = *reinterpret_cast<const bf16x8*>(vrow + ((h * 4 + g) ^ v_swizzle((dt + 1) * 16 + r)) * 8);
        }
#pragma unroll
        for (int x = 0; x < PF_UNITS; ++x) {
            if (!u[x].active) continue;
#pragma unroll
            for (int h = 0; h < 2; ++h) u[x].c.o[dt] = mfma_16x16x32(vf[dt & 1][h], pv[x][h], u[x].c.o[dt]);
        }
    }
}

// grid (query tiles, nkv * head groups, sequences)
// Two waves on a SIMD, where the head size lets the registers fit without spilling: a second block on the
// compute unit runs while one waits at a barrier or for LDS.
#if PALM_HEAD_DIM <= 128
#define PF_WAVES_PER_SIMD __attribute__((amdgpu_waves_per_eu(2)))
#else
#define PF_WAVES_PER_SIMD
#endif
__global__ __launch_bounds__(PF_THREADS) PF_WAVES_PER_SIMD void attention_prefill_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_start, const int* __restrict__ seq_new, const int* __restrict__ cu_new, int nh,
    int nkv, float scale_log2, int window, int qb, int hg, bf16_t* __restrict__ out) {
    constexpr int K_TILE = PAGE_TOKENS * K_STRIDE, V_TILE = HD * V_STRIDE;
    // Head sizes whose pages fit twice keep two pages of K and of V^T in LDS: while one is used the next is laid
    // down beside it, and one barrier a page is enough.  Larger heads share one buffer between K and V^T.
    __shared__ __attribute__((aligned(16))) bf16_t k_lds[PF_SHARE ? (V_TILE > K_TILE ? V_TILE : K_TILE) : 2 * K_TILE];
    __shared__ __attribute__((aligned(16))) bf16_t v_own[PF_SHARE ? 8 : 2 * V_TILE];
    bf16_t* v_lds = PF_SHARE ? k_lds : v_own;

    const int b = blockIdx.z;
    const int G = nh / nkv, n_hg = (G + hg - 1) / hg;
    const int kvh = blockIdx.x / n_hg, hgi = blockIdx.x % n_hg;       // the kv head runs fastest over the blocks, see the launch
    const int n_new = seq_new[b];
    // the block's sub-tiles of 16 queries: number s is, for even s, sub-tile f = first + s / 2 from the front, for
    // odd s its partner n16 - 1 - f from the back (none if f is the middle one); a single sub-tile a block (eight
    // heads a group) just counts from the back, the long ones first
    const int subs = qb / 16, n16 = (n_new + 15) / 16;
    const int first_front = blockIdx.y * (subs > 1 ? subs / 2 : 1);
    if (subs > 1 ? 2 * first_front > n16 - 1 : first_front >= n16) return;
    auto sub_tile = [&](int sub) -> int {                       // the sub-tile's index, or -1
        if (subs == 1) return n16 - 1 - first_front;
        const int f = first_front + sub / 2, partner = n16 - 1 - f;
        if (f > partner) return -1;
        return (sub & 1) ? (partner > f ? partner : -1) : f;
    };
    const int lane = threadIdx.x % WAVE, r = lane % 16, g = lane / 16;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);      // the same in every lane: what follows from it stays scalar
    const int start = seq_start[b];
    const int seq_tail = start + n_new - 1;                     // the sequence's last key
    const int heads_here = min(hg, G - hgi * hg);
    const int n_units = heads_here * subs;
    const int* pages = block_table + (size_t)seq_slot[b] * max_pages;

    Unit u[PF_UNITS];
#pragma unroll
    for (int x = 0; x < PF_UNITS; ++x) {
        const int unit = wave + x * PF_WAVES;
        const int tile16 = unit < n_units ? sub_tile(unit / heads_here) : -1;
        u[x].live = tile16 >= 0;
        const int un = u[x].live ? unit : 0;
        const int q_first = max(tile16, 0) * 16;                   // the unit's first query, within the step
        const int qi = q_first + r;
        u[x].page_hi = (start + min(q_first + 15, n_new - 1)) / PAGE_TOKENS;
        u[x].page_lo = window > 0 ? max(0, start + q_first - window + 1) / PAGE_TOKENS : 0;
        u[x].head = kvh * G + hgi * hg + un % heads_here;
        u[x].valid = u[x].live && qi < n_new;
        const int qc = min(qi, n_new - 1);
        u[x].pos = start + qc;
        u[x].first = window > 0 ? max(0, u[x].pos - window + 1) : 0;
        u[x].row = (size_t)cu_new[b] + qc;
        load_query(q + (u[x].row * nh + u[x].head) * HD, true, g, u[x].qv);
        u[x].c.m = -INFINITY;
        u[x].c.l = 0.f;
        u[x].weights = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dt = 0; dt < DTILES; ++dt) u[x].c.o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // the pages any of the block's sub-tiles sees (the same for all waves)
    int p_lo = 0x7fffffff, p_hi = -1;
    for (int sub = 0; sub < subs; ++sub) {
        const int tile16 = sub_tile(sub);
        if (tile16 < 0) continue;
        p_hi = max(p_hi, (start + min(tile16 * 16 + 15, n_new - 1)) / PAGE_TOKENS);
        p_lo = min(p_lo, window > 0 ? max(0, start + tile16 * 16 - window + 1) / PAGE_TOKENS : 0);
    }
    PagePrefetch pf;
    PageSources sources;
    {
        const size_t base = ((size_t)pages[p_lo] * nkv + kvh) * PAGE_TOKENS * HD;
        if constexpr (PF_DMA) {
            sources = page_sources();
            page_into_lds(k_cache + base, v_cache + base, sources, k_lds, v_lds);
        } else {
            prefetch_keys(k_cache + base, pf);
            prefetch_values(v_cache + base, pf);
        }
    }
    // is every key of page p visible to every column of this wave that takes part?  (also marks who does)
    auto page_is_interior = [&](int p) -> bool {
        bool inside = true;
#pragma unroll
        for (int x = 0; x < PF_UNITS; ++x) {
            u[x].active = u[x].live && p >= u[x].page_lo && p <= u[x].page_hi;
            inside = inside && (!u[x].active || (u[x].first <= p * PAGE_TOKENS && u[x].pos >= p * PAGE_TOKENS + PAGE_TOKENS - 1));
        }
        return __all(inside);
    };
    if constexpr (!PF_SHARE) {
        if constexpr (PF_DMA) {
            lds_loads_done();
        } else {
            stage_keys(pf, k_lds);
            stage_values(pf, v_lds);
        }
        __syncthreads();
        for (int p = p_lo; p <= p_hi; ++p) {
            const int buf = (p - p_lo) & 1;
            const bool more = p < p_hi;
            if (seq_tail - p * PAGE_TOKENS < PAGE_TOKENS - 1) {     // the sequence's last page (no page follows it)
                blank_values_after(v_lds + buf * V_TILE, seq_tail - p * PAGE_TOKENS);
                __syncthreads();
            }
            if (more) {                                         // in flight while this page is used
                const size_t next = ((size_t)pages[p + 1] * nkv + kvh) * PAGE_TOKENS * HD;
                if constexpr (PF_DMA) {     // straight into the other buffer, whose last readers passed the barrier a page ago
                    page_into_lds(k_cache + next, v_cache + next, sources, k_lds + (buf ^ 1) * K_TILE, v_lds + (buf ^ 1) * V_TILE);
                } else {
                    prefetch_keys(k_cache + next, pf);
                    prefetch_values(v_cache + next, pf);
                }
            }
            bf16x8 pv[PF_UNITS][2];
            float alpha[PF_UNITS];
            const bool interior = page_is_interior(p);
            unit_scores(k_lds + buf * K_TILE, u, p * PAGE_TOKENS, scale_log2, r, g, interior, pv, alpha);
            bool moved = false;
#pragma unroll
            for (int x = 0; x < PF_UNITS; ++x) moved = moved || alpha[x] != 1.0f;
            unit_values(v_lds + buf * V_TILE, u, r, g, pv, alpha, __any(moved));
            if constexpr (!PF_DMA) {
                if (more) {                                     // the other buffer's last readers passed the barrier a page ago
                    stage_keys(pf, k_lds + (buf ^ 1) * K_TILE);
                    stage_values(pf, v_lds + (buf ^ 1) * V_TILE);
                }
            }
            if constexpr (PF_DMA) lds_loads_done();
            __syncthreads();
        }
    } else {
        for (int p = p_lo; p <= p_hi; ++p) {
            const bool more = p < p_hi;
            const size_t next = more ? ((size_t)pages[p + 1] * nkv + kvh) * PAGE_TOKENS * HD : 0;
            bf16x8 pv[PF_UNITS][2];
            float alpha[PF_UNITS];
            __syncthreads();                                    // everyone is done with the previous page
            stage_keys(pf, k_lds);
            __syncthreads();
            if (more) prefetch_keys(k_cache + next, pf);        // in flight while this page is used
            const bool interior = page_is_interior(p);
            unit_scores(k_lds, u, p * PAGE_TOKENS, scale_log2, r, g, interior, pv, alpha);
            bool moved = false;
#pragma unroll
            for (int x = 0; x < PF_UNITS; ++x) moved = moved || alpha[x] != 1.0f;
            const bool rescale = __any(moved);
            __syncthreads();
            stage_values(pf, v_lds);
            __syncthreads();
            if (seq_tail - p * PAGE_TOKENS < PAGE_TOKENS - 1) {
                blank_values_after(v_lds, seq_tail - p * PAGE_TOKENS);
                __syncthreads();
            }
            unit_values(v_lds, u, r, g, pv, alpha, rescale);
            if (more) prefetch_values(v_cache + next, pf);
        }
    }

#pragma unroll
    for (int x = 0; x < PF_UNITS; ++x) {
        const float l = u[x].weights[0];
        if (u[x].valid) {
            const float inv = 1.0f / l;
            bf16_t* o = out + (u[x].row * nh + u[x].head) * HD;
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt) {               // the lane's four elements of a tile lie side by side: one store
                uint2 four;
                four.x = (uint32_t)f32_to_bf16(u[x].c.o[dt][0] * inv).bits | ((uint32_t)f32_to_bf16(u[x].c.o[dt][1] * inv).bits << 16);
                four.y = (uint32_t)f32_to_bf16(u[x].c.o[dt][2] * inv).bits | ((uint32_t)f32_to_bf16(u[x].c.o[dt][3] * inv).bits << 16);
                *reinterpret_cast<uint2*>(o + dt * 16 + 4 * g) = four;
            }
        }
    }
}

// ---- prefill for the head sizes whose pages go straight into LDS (64, 128) --------------------------
// The same block of four waves, eight units and pages staged once in LDS, arranged so that the page loop is one
// stretch of arithmetic without a branch around any matrix instruction:
//  * a wave's two units lie next to each other (the same head's neighbouring 16 queries where a kv head has four
//    query heads), so both see almost the same pages, and there is no unit to switch on and off: a page that a unit
//    does not see at all is simply a page whose every key is masked for it;
//  * a block has one tile of queries, and a late tile has many more pages to walk than an early one.  Where the
//    launch has more blocks than the chip holds at once, the long ones simply go first.  Where all its blocks run at
//    once (a prompt of a few thousand tokens), two share a compute unit, and the numbering makes blocks k and k + 256,
//    which the dispatcher is expected to place together, a tile from the back and its partner from the front, so
//    that every unit gets about the same work;
//  * the scores come out of the matrix cores already taken against the column's reference (the accumulator starts at
//    minus the reference instead of zero; with queries that come multiplied by scale * log2(e), q_prescaled, no
//    multiplication is left either), so a weight is one exp2 and one rounding;
//  * the reference follows the running maximum only when a column's scores have risen more than 2^PF_LAZY_LOG2 above
//    it.  Whether any column of the wave has to move is one vote over the lanes' own sixteen scores; the exchange
//    between the four lanes of a column, the shift and the rescaling of the outputs stand behind that vote, off the
//    usual path;
//  * STAGES pages of K and V^T lie in LDS, STAGES - 1 of them on their way while one is used: two where many blocks
//    share a compute unit, four where a short prompt leaves a unit one block, whose loads then need a longer lead.
//    The barrier between pages waits for LDS and for the one page that is needed next, not for the younger loads.
template <int N> __device__ __forceinline__ void wait_for_all_but_the_youngest_loads() {
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));          // s_waitcnt vmcnt(N)
}
__device__ __forceinline__ void page_barrier() {     // LDS reads done, then the block's barrier; loads stay in flight
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

struct PairedUnit {           // one (head, 16 query positions): the wave's share of it
    bool live, valid;         // the wave has such a unit; this lane's column is a real query
    int pos, first;           // the column's position and the first key it sees
    size_t row;               // the column's row in q and out
    int head;
    float m;                  // the reference the column's weights are taken against (-inf before its first key)
    bf16x8 qv[KSTEPS];
    f32x4 o[DTILES];
    f32x4 weights;            // the sum of the column's weights, four times
};

// masked (the same in every lane): some column of the wave does not see every key of the page
constexpr int VALUES_AHEAD = DTILES / 2;       // value tiles whose fragments are asked for before the weights are made
template <bool PRESCALED>
__device__ __forceinline__ void paired_page(const bf16_t* k_lds, const bf16_t* v_lds, PairedUnit (&u)[PF_UNITS], int page_first_key,
                                            float scale_log2, int r, int g, bool masked) {
    f32x4 s[PF_UNITS][4];
    float sub[PF_UNITS];
#pragma unroll
    for (int x = 0; x < PF_UNITS; ++x) sub[x] = u[x].m == -INFINITY ? 0.f : u[x].m;
    // A fragment read from LDS takes longer than the few matrix instructions it feeds, so fragments are asked for
    // well ahead: all of a page's keys at once (the weights' and values' registers are free then), and the values
    // as soon as the scores are done, so that they arrive while the weights are made.
    bf16x8 kf[4][KSTEPS];
#pragma unroll
    for (int t = 0; t < 4; ++t) read_key_fragments(k_lds, t, r, g, kf[t]);
#pragma unroll
    for (int t = 0; t < 4; ++t) {
#pragma unroll
        for (int x = 0; x < PF_UNITS; ++x) {
            const float from = PRESCALED ? -sub[x] : 0.f;
            f32x4 acc = f32x4{from, from, from, from};
#pragma unroll
            for (int j = 0; j < KSTEPS; ++j) acc = mfma_16x16x32(kf[t][j], u[x].qv[j], acc);
            s[x][t] = acc;
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    bf16x8 vf[DTILES][2];
#pragma unroll
    for (int dt = 0; dt < VALUES_AHEAD; ++dt) {
        const int row = dt * 16 + r;
#pragma unroll
        for (int h = 0; h < 2; ++h) vf[dt][h] = *reinterpret_cast<const bf16x8*>(v_lds + row * V_STRIDE + ((h * 4 + g) ^ v_swizzle(row)) * 8);
    }
    __builtin_amdgcn_sched_barrier(0);

    bool vote = masked;
    float mx[PF_UNITS];
#pragma unroll
    for (int x = 0; x < PF_UNITS; ++x) {
        if (!PRESCALED) {
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) s[x][t][i] = fmaf(s[x][t][i], scale_log2, -sub[x]);
        }
        if (masked) {
            const int lo = u[x].first - page_first_key, hi = u[x].pos - page_first_key;
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int key = tile_key(t, 4 * g + i);
                    s[x][t][i] = (key >= lo && key <= hi) ? s[x][t][i] : -INFINITY;
                }
        }
        float top = s[x][0][0];
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) top = fmaxf(top, s[x][t][i]);
        mx[x] = top;
        vote = vote || top > PF_LAZY_LOG2 || u[x].m == -INFINITY;
    }
    if (__any(vote)) {
#pragma unroll
        for (int x = 0; x < PF_UNITS; ++x) {
            float top = mx[x];                                          // of the column: its four lanes agree
            top = fmaxf(top, __shfl_xor(top, 16, WAVE));
            top = fmaxf(top, __shfl_xor(top, 32, WAVE));
            const bool fresh = u[x].m == -INFINITY;                     // no key yet: outputs and sums are still zero
            const bool jump = top > PF_LAZY_LOG2 || (fresh && top > -INFINITY);
            const float shift = jump ? top : 0.f;
            const float alpha = jump && !fresh ? exp2_weight(-top) : 1.0f;
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) s[x][t][i] -= shift;
            if (jump) u[x].m = sub[x] + top;
            if (__any(alpha != 1.0f)) {
#pragma unroll
                for (int dt = 0; dt < DTILES; ++dt) u[x].o[dt] = u[x].o[dt] * alpha;
                u[x].weights = u[x].weights * alpha;
            }
        }
    }
    bf16x8 pv[PF_UNITS][2];
#pragma unroll
    for (int x = 0; x < PF_UNITS; ++x)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int e = 0; e < 8; ++e) pv[x][h][e] = (__bf16)exp2_weight(s[x][2 * h + e / 4][e % 4]);

    // the sum of a column's weights comes from the matrix cores too: a row of ones in place of a row of V^T
    bf16x8 ones;
#pragma unroll
    for (int e = 0; e < 8; ++e) ones[e] = (__bf16)1.0f;
#pragma unroll
    for (int x = 0; x < PF_UNITS; ++x)
#pragma unroll
        for (int h = 0; h < 2; ++h) u[x].weights = mfma_16x16x32(ones, pv[x][h], u[x].weights);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int dt = VALUES_AHEAD; dt < DTILES; ++dt) {        // the rest of the values, now that the scores' registers are free
        const int row = dt * 16 + r;
#pragma unroll
        for (int h = 0; h < 2; ++h) vf[dt][h] = *reinterpret_cast<const bf16x8*>(v_lds + row * V_STRIDE + ((h * 4 + g) ^ v_swizzle(row)) * 8);
    }
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int x = 0; x < PF_UNITS; ++x) u[x].o[dt] = mfma_16x16x32(vf[dt][h], pv[x][h], u[x].o[dt]);
}

template <int STAGES, bool PRESCALED>
__global__ __launch_bounds__(PF_THREADS) PF_WAVES_PER_SIMD void attention_prefill_paired_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_start, const int* __restrict__ seq_new, const int* __restrict__ cu_new, int nh,
    int nkv, float scale_log2, int window, int qb, int hg, int partners_follow, bf16_t* __restrict__ out) {
    if constexpr (PF_DMA) {
        constexpr int K_TILE = PAGE_TOKENS * K_STRIDE, V_TILE = HD * V_STRIDE;
        constexpr int PAGE_LOADS = 2 * PF_LOADS;                    // a wave's instructions for one page of K and V^T
        __shared__ __attribute__((aligned(16))) bf16_t k_lds[STAGES * K_TILE];
        __shared__ __attribute__((aligned(16))) bf16_t v_lds[STAGES * V_TILE];

        const int b = blockIdx.z;
        const int G = nh / nkv, n_hg = (G + hg - 1) / hg;
        const int kvh = blockIdx.x / n_hg, hgi = blockIdx.x % n_hg;   // the kv head runs fastest over the blocks, see the launch
        const int n_new = seq_new[b];
        const int subs = qb / 16, n_q = (n_new + qb - 1) / qb;        // tiles of qb queries in this sequence
        if ((int)blockIdx.y >= n_q) return;
        // first the tiles from the back (the long ones), the last first; then, where the launch asks for it, their
        // partners from the front in the same order, else the rest from the back too
        const int half = (n_q + 1) / 2, y = blockIdx.y;
        const int tile = y < half || !partners_follow ? n_q - 1 - y : y - half;
        const int lane = threadIdx.x % WAVE, r = lane % 16, g = lane / 16;
        const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
        const int start = seq_start[b];
        const int seq_tail = start + n_new - 1;                       // the sequence's last key
        const int heads_here = min(hg, G - hgi * hg);
        const int n_units = heads_here * subs;
        const int* pages = block_table + (size_t)seq_slot[b] * max_pages;
        const PageSources sources = page_sources();

        {
            const int tile_first = tile * qb;                         // the tile's first query, within the step
            PairedUnit u[PF_UNITS];
#pragma unroll
            for (int x = 0; x < PF_UNITS; ++x) {
                const int unit = wave + x * PF_WAVES;
                const int sub = unit / heads_here;                    // the unit's 16 queries within the tile
                const int q_first = tile_first + sub * 16;
                u[x].live = unit < n_units && q_first < n_new;
                const int qi = q_first + r;
                u[x].head = kvh * G + hgi * hg + (unit < n_units ? unit % heads_here : 0);
                u[x].valid = u[x].live && qi < n_new;
                const int qc = min(qi, n_new - 1);
                u[x].pos = start + qc;
                u[x].first = window > 0 ? max(0, u[x].pos - window + 1) : 0;
                u[x].row = (size_t)cu_new[b] + qc;
                load_query(q + (u[x].row * nh + u[x].head) * HD, true, g, u[x].qv);
                u[x].m = -INFINITY;
                u[x].weights = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int dt = 0; dt < DTILES; ++dt) u[x].o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
            // the pages any query of the tile sees (the same for all waves)
            const int tile_last = min(tile_first + qb - 1, n_new - 1);
            const int p_hi = (start + tile_last) / PAGE_TOKENS;
            const int p_lo = window > 0 ? max(0, start + tile_first - window + 1) / PAGE_TOKENS : 0;
            auto load_page = [&](int p) {
                const size_t at = ((size_t)pages[p] * nkv + kvh) * PAGE_TOKENS * HD;
                const int stage = (p - p_lo) % STAGES;
                page_into_lds(k_cache + at, v_cache + at, sources, k_lds + stage * K_TILE, v_lds + stage * V_TILE);
            };
            // is every key of page p visible to every column of this wave?
            auto interior = [&](int p) -> bool {
                bool inside = true;
#pragma unroll
                for (int x = 0; x < PF_UNITS; ++x)
                    inside = inside && (!u[x].live || (u[x].first <= p * PAGE_TOKENS && u[x].pos >= p * PAGE_TOKENS + PAGE_TOKENS - 1));
                return __all(inside);
            };
            wait_for_all_but_the_youngest_loads<0>();                 // the queries
#pragma unroll
            for (int ahead = 0; ahead < STAGES - 1; ++ahead)
                if (p_lo + ahead <= p_hi) load_page(p_lo + ahead);
            // the first page has landed when at most the pages after it are on their way
            if constexpr (STAGES > 2) {
                const int young = min(p_hi - p_lo, STAGES - 2);
                if (young >= 2) wait_for_all_but_the_youngest_loads<2 * PAGE_LOADS>();
                else if (young == 1) wait_for_all_but_the_youngest_loads<PAGE_LOADS>();
                else wait_for_all_but_the_youngest_loads<0>();
            } else {
                wait_for_all_but_the_youngest_loads<0>();
            }
            page_barrier();
            for (int p = p_lo; p <= p_hi; ++p) {
                const int stage = (p - p_lo) % STAGES;
                if (p + STAGES - 1 <= p_hi) load_page(p + STAGES - 1);      // into the stage whose readers passed the barrier a page ago
                bf16_t* v_page = v_lds + stage * V_TILE;
                if (seq_tail - p * PAGE_TOKENS < PAGE_TOKENS - 1) {          // the sequence's last page: no page follows it
                    blank_values_after(v_page, seq_tail - p * PAGE_TOKENS);
                    __syncthreads();
                }
                paired_page<PRESCALED>(k_lds + stage * K_TILE, v_page, u, p * PAGE_TOKENS, scale_log2, r, g, !interior(p));
                // the next page has landed when at most the pages after it are on their way
                if constexpr (STAGES > 2) {
                    const int young = min(p_hi, p + STAGES - 1) - (p + 1);
                    if (young >= 2) wait_for_all_but_the_youngest_loads<2 * PAGE_LOADS>();
                    else if (young == 1) wait_for_all_but_the_youngest_loads<PAGE_LOADS>();
                    else wait_for_all_but_the_youngest_loads<0>();
                } else {
                    wait_for_all_but_the_youngest_loads<0>();
                }
                page_barrier();
            }
#pragma unroll
            for (int x = 0; x < PF_UNITS; ++x) {
                if (u[x].valid) {
                    const float inv = 1.0f / u[x].weights[0];
                    bf16_t* o = out + (u[x].row * nh + u[x].head) * HD;
#pragma unroll
                    for (int dt = 0; dt < DTILES; ++dt) {           // the lane's four elements of a tile lie side by side: one store
                        uint2 four;
                        four.x = (uint32_t)f32_to_bf16(u[x].o[dt][0] * inv).bits | ((uint32_t)f32_to_bf16(u[x].o[dt][1] * inv).bits << 16);
                        four.y = (uint32_t)f32_to_bf16(u[x].o[dt][2] * inv).bits | ((uint32_t)f32_to_bf16(u[x].o[dt][3] * inv).bits << 16);
                        *reinterpret_cast<uint2*>(o + dt * 16 + 4 * g) = four;
                    }
                }
            }
        }
    }
}

// q_prescaled: the queries come multiplied by scale * log2(e) already (by the pass that rounds them), so a score is
// the exponent of its weight as it leaves the matrix cores; `scale` is then not applied again.
PALM_API int palm_attention_prefill(hipStream_t stream, const void* q, const void* k_cache, const void* v_cache,
                                    const int* block_table, int max_pages, const int* seq_slot, const int* seq_start,
                                    const int* seq_new, const int* cu_new, int n_seqs, int max_new, int nh, int nkv,
                                    int hd, float scale, int window, int q_prescaled, void* out) {
    PALM_CHECK(hd == HD, "attention_prefill: this library was built for head size %d, not %d", HD, hd);
    PALM_CHECK(n_seqs >= 0 && max_new >= 0 && nh > 0 && nkv > 0 && nh % nkv == 0,
               "attention_prefill: seqs=%d max_new=%d heads=%d kv=%d", n_seqs, max_new, nh, nkv);
    PALM_CHECK(window >= 0 && max_pages > 0, "attention_prefill: window=%d max_pages=%d", window, max_pages);
    if (n_seqs == 0 || max_new == 0) return 0;
    const int G = nh / nkv;
    constexpr int UNITS = PF_UNITS * PF_WAVES;                 // (head, 16 queries) units a block holds
    const int hg = G < UNITS ? G : UNITS;                      // query heads of the group served by one block
    const int qb = 16 * (UNITS / hg > 0 ? UNITS / hg : 1);     // query positions in a tile
    const int n_hg = (G + hg - 1) / hg;
    PALM_CHECK(nkv * n_hg <= 65535 && n_seqs <= 65535, "attention_prefill: grid too large");
    const float scale_log2 = q_prescaled ? 1.0f : scale * LOG2E;
    // Blocks are handed to the chip's eight dies in turn by their number, and each die has an L2 of its own.  With
    // the kv head as the fastest index, the blocks that a die gets belong to few kv heads (one, with eight of
    // them), whose keys and values then stay in that die's L2 for all the query tiles that read them.
    if constexpr (PF_DMA) {
        const int n_q = (max_new + qb - 1) / qb;
        PALM_CHECK(n_q <= 65535, "attention_prefill: %d new tokens are more than one launch takes", max_new);
        dim3 grid(nkv * n_hg, n_q, n_seqs);
        const long long blocks = (long long)grid.x * grid.y * grid.z;
        // four pages in LDS leave a compute unit room for one block: where the launch has no second block for it anyway
        const bool few = blocks <= 256;
        const int partners_follow = blocks <= 512 && n_seqs == 1;     // all blocks run at once, two a unit
#define PALM_PAIRED(STAGES, PRE) attention_prefill_paired_kernel<STAGES, PRE><<<grid, PF_THREADS, 0, stream>>>( \
        (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, max_pages, seq_slot, seq_start, seq_new, \
        cu_new, nh, nkv, scale_log2, window, qb, hg, partners_follow, (bf16_t*)out)
        if (few) { if (q_prescaled) PALM_PAIRED(4, true); else PALM_PAIRED(4, false); }
        else { if (q_prescaled) PALM_PAIRED(2, true); else PALM_PAIRED(2, false); }
#undef PALM_PAIRED
        PALM_LAUNCHED();
        return 0;
    }
    PALM_CHECK(!q_prescaled, "attention_prefill: head size %d takes its queries as they are and applies the scale itself", HD);
    const int n16 = (max_new + 15) / 16, subs = qb / 16;
    const int n_tiles = subs > 1 ? ((n16 + 1) / 2 + subs / 2 - 1) / (subs / 2) : n16;
    PALM_CHECK(n_tiles <= 65535, "attention_prefill: %d new tokens are more than one launch takes", max_new);
    dim3 grid(nkv * n_hg, n_tiles, n_seqs);
    attention_prefill_kernel<<<grid, PF_THREADS, 0, stream>>>((const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache,
                                                             block_table, max_pages, seq_slot, seq_start, seq_new, cu_new, nh,
                                                             nkv, scale_log2, window, qb, hg, (bf16_t*)out);
    PALM_LAUNCHED();
    return 0;
}

PALM_API int palm_attention_prefill_takes_prescaled() { return PF_DMA ? 1 : 0; }
