// Embedding gather, RMSNorm (with the residual add fused in), SwiGLU and element type casts.
//
// Formulas follow the reference: embedding rows widened to 32-bit (engine/engine.cpp:332-357);
// y = x * (1/sqrt(mean(x^2) + eps)) * w with the statistics in 32-bit (kernels/norm.cpp:13-31,
// engine/cuda_ops.cu:114-138); fused residual update then norm (engine/cuda_ops.cu:140-170);
// out = g / (1 + exp(-g)) * u over merged [gate | up] rows (engine/cuda_ops.cu:100-112).
#include "common.h"

PALM_DEFINE_LAST_ERROR()

PALM_API int palm_page_tokens() { return PAGE_TOKENS; }

// ---- embedding ------------------------------------------------------------------------------------
// One block per token.  An id outside the table gives a row of NaN: visible, and no read out of bounds.
template <typename TW>
__global__ void embed_kernel(const TW* __restrict__ table, const int* __restrict__ ids, float* __restrict__ out,
                             int hidden, int vocab) {
    const int t = blockIdx.x;
    const int id = ids[t];
    float* dst = out + (size_t)t * hidden;
    if (id < 0 || id >= vocab) {
        for (int d = threadIdx.x; d < hidden; d += blockDim.x) dst[d] = NAN;
        return;
    }
    const TW* src = table + (size_t)id * hidden;
    for (int d = threadIdx.x; d < hidden; d += blockDim.x) dst[d] = to_float(src[d]);
}

PALM_API int palm_embed(hipStream_t stream, const void* table, int table_dtype, const int* ids, int n_tokens,
                        int hidden, int vocab, float* out) {
    PALM_CHECK(n_tokens >= 0 && hidden > 0 && vocab > 0, "embed: n_tokens=%d hidden=%d vocab=%d", n_tokens, hidden, vocab);
    if (n_tokens == 0) return 0;
    PALM_DTYPE_SWITCH(table_dtype, TW,
        embed_kernel<TW><<<n_tokens, 256, 0, stream>>>((const TW*)table, ids, out, hidden, vocab));
    PALM_LAUNCHED();
    return 0;
}

// ---- RMSNorm --------------------------------------------------------------------------------------
// One block per output row.  src row = rows ? rows[r] : r.  v = x[src] (+ delta[src]).  If update_x the
// sum is written back to x (only without `rows`), so the residual stream is updated and normed in one
// pass over it.  Statistics and products in 32-bit; the product order is (v * r) * w.
// delta may be `planes` planes of partial sums, plane_stride elements apart (a projection that cut its K into
// ranges); they are added one after the other, plane 0 first.
constexpr int NORM_MAX_PLANES = 4;

template <typename TX, typename TD, typename TO>
__global__ void rmsnorm_kernel(TX* __restrict__ x, const TD* __restrict__ delta, int planes, size_t plane_stride,
                               const float* __restrict__ w,
                               const int* __restrict__ rows, TO* __restrict__ out, int width, float eps,
                               int update_x) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t src = rows ? (size_t)rows[r] : (size_t)r;
    TX* xr = x + src * width;
    const TD* dr = delta ? delta + src * width : nullptr;
    float ss = 0.f;
    for (int d = threadIdx.x; d < width; d += blockDim.x) {
        float v = to_float(xr[d]);
        if (dr) for (int p = 0; p < planes; ++p) v += to_float(dr[p * plane_stride + d]);
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)width + eps);
    TO* o = out + (size_t)r * width;
    for (int d = threadIdx.x; d < width; d += blockDim.x) {
        float v = to_float(xr[d]);
        if (dr) for (int p = 0; p < planes; ++p) v += to_float(dr[p * plane_stride + d]);
        if (update_x) xr[d] = from_float<TX>(v);
        o[d] = from_float<TO>(v * inv * w[d]);
    }
}

// The same, for widths that are a multiple of four and fit the block's registers: every thread reads its
// elements once, four at a time, all reads issued before the first is used (a decode step's rows are few and
// the kernel's time is the latency of its reads, so reads that wait for each other are what must be avoided).
__device__ inline void load4(const float* p, float (&v)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ inline void load4(const bf16_t* p, float (&v)[4]) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
    v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
}
__device__ inline void store4(float* p, const float (&v)[4]) { *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]); }
__device__ inline void store4(bf16_t* p, const float (&v)[4]) {
    uint2 t;
    t.x = (uint32_t)f32_to_bf16(v[0]).bits | ((uint32_t)f32_to_bf16(v[1]).bits << 16);
    t.y = (uint32_t)f32_to_bf16(v[2]).bits | ((uint32_t)f32_to_bf16(v[3]).bits << 16);
    *reinterpret_cast<uint2*>(p) = t;
}

template <typename TX, typename TD, typename TO, int ITERS, int PLANES>
__global__ void rmsnorm_fast_kernel(TX* __restrict__ x, const TD* __restrict__ delta, int planes, size_t plane_stride,
                                    const float* __restrict__ w,
                                    const int* __restrict__ rows, TO* __restrict__ out, int width, float eps,
                                    int update_x) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t src = rows ? (size_t)rows[r] : (size_t)r;
    TX* xr = x + src * width;
    const TD* dr = delta ? delta + src * width : nullptr;
    float v[ITERS][4], d[PLANES][ITERS][4], wt[ITERS][4];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int i = (it * blockDim.x + threadIdx.x) * 4;
        const int at = i < width ? i : 0;                   // a thread beyond the row reads its start and adds nothing
        load4(xr + at, v[it]);
        load4(w + at, wt[it]);
        if (dr) {
#pragma unroll
            for (int p = 0; p < PLANES; ++p) load4(dr + (size_t)min(p, planes - 1) * plane_stride + at, d[p][it]);   // an absent plane reads the last one and adds nothing
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const bool in = (it * blockDim.x + threadIdx.x) * 4 < width;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (dr) {
#pragma unroll
                for (int p = 0; p < PLANES; ++p) v[it][e] += p < planes ? d[p][it][e] : 0.f;
            }
            if (in) ss += v[it][e] * v[it][e];
        }
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)width + eps);
    TO* o = out + (size_t)r * width;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int i = (it * blockDim.x + threadIdx.x) * 4;
        if (i >= width) continue;
        if (update_x) store4(xr + i, v[it]);
        float y[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) y[e] = v[it][e] * inv * wt[it][e];
        store4(o + i, y);
    }
}

template <typename TX, typename TD, typename TO>
static bool launch_rmsnorm_fast(hipStream_t stream, void* x, const void* delta, int planes, size_t plane_stride,
                                const float* weight, float eps,
                                const int* rows, int n_out_rows, int width, void* out, int update_x) {
    if (width % 4 != 0 || width > 32768) return false;
    const int quads = width / 4;
    int iters = quads <= 256 ? 1 : (quads <= 512 ? 2 : (quads <= 1024 ? 4 : 8));
    if (planes > 1 && iters > 4) {                          // eight quads of several planes do not fit a thread's registers:
        if (quads > 4096) return false;                     // more threads with four quads each, as far as a block goes
        iters = 4;
    }
    int threads = (quads + iters - 1) / iters;
    threads = (threads + WAVE - 1) / WAVE * WAVE;
    if (threads > 1024) return false;
#define PALM_NORM_CASE(IT) case IT: \
        if (planes > 1) rmsnorm_fast_kernel<TX, TD, TO, IT, NORM_MAX_PLANES><<<n_out_rows, threads, 0, stream>>>( \
            (TX*)x, (const TD*)delta, planes, plane_stride, weight, rows, (TO*)out, width, eps, update_x); \
        else rmsnorm_fast_kernel<TX, TD, TO, IT, 1><<<n_out_rows, threads, 0, stream>>>( \
            (TX*)x, (const TD*)delta, 1, plane_stride, weight, rows, (TO*)out, width, eps, update_x); \
        break;
    switch (iters) { PALM_NORM_CASE(1) PALM_NORM_CASE(2) PALM_NORM_CASE(4) PALM_NORM_CASE(8) }
#undef PALM_NORM_CASE
    return true;
}

// delta_planes > 1: delta is [delta_planes, rows of x, width] float32.
PALM_API int palm_rmsnorm(hipStream_t stream, void* x, int x_dtype, const void* delta, int delta_dtype, int delta_planes,
                          const float* weight, float eps, const int* rows, int n_out_rows, int width,
                          void* out, int out_dtype, int update_x, long long x_rows) {
    PALM_CHECK(n_out_rows >= 0 && width > 0, "rmsnorm: rows=%d width=%d", n_out_rows, width);
    PALM_CHECK(!(update_x && rows), "rmsnorm: the residual cannot be updated through a row selection");
    PALM_CHECK(!(update_x && !delta), "rmsnorm: update_x without a delta has nothing to add");
    PALM_CHECK(delta_planes >= 1 && delta_planes <= NORM_MAX_PLANES, "rmsnorm: %d planes of delta (at most %d)",
               delta_planes, NORM_MAX_PLANES);
    PALM_CHECK(delta_planes == 1 || (delta && delta_dtype == PALM_F32), "rmsnorm: planes of delta are float32");
    if (n_out_rows == 0) return 0;
    const size_t plane_stride = (size_t)x_rows * width;
    {
        bool done = false;
        PALM_DTYPE_SWITCH(x_dtype, TX, PALM_DTYPE_SWITCH(delta_dtype, TD, PALM_DTYPE_SWITCH(out_dtype, TO,
            done = launch_rmsnorm_fast<TX, TD, TO>(stream, x, delta, delta_planes, plane_stride, weight, eps, rows, n_out_rows,
                                                   width, out, update_x))));
        if (done) { PALM_LAUNCHED(); return 0; }
    }
    const int threads = width >= 1024 ? 256 : (width >= 256 ? 128 : 64);
    PALM_DTYPE_SWITCH(x_dtype, TX, PALM_DTYPE_SWITCH(delta_dtype, TD, PALM_DTYPE_SWITCH(out_dtype, TO,
        rmsnorm_kernel<TX, TD, TO><<<n_out_rows, threads, 0, stream>>>(
            (TX*)x, (const TD*)delta, delta_planes, plane_stride, weight, rows, (TO*)out, width, eps, update_x))));
    PALM_LAUNCHED();
    return 0;
}

// Rows that a product left without their norm's factor (linear_mfma.hip, RowNorm): out = a * f(row),
// f = 1 / sqrt(sum of the row's pieces / width + eps).  Only for a reader that cannot apply the factor itself.
template <typename T>
__global__ void scale_rows_kernel(const T* __restrict__ a, const float* __restrict__ ss, int pieces, int n_rows,
                                  float eps, int width, T* __restrict__ out) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    float sum = 0.f;
    for (int p = threadIdx.x; p < pieces; p += blockDim.x) sum += ss[(size_t)r * pieces + p];
    sum = block_sum(sum, scratch);
    const float f = 1.0f / sqrtf(sum / (float)width + eps);
    for (int d = threadIdx.x; d < width; d += blockDim.x)
        out[(size_t)r * width + d] = from_float<T>(to_float(a[(size_t)r * width + d]) * f);
}

PALM_API int palm_scale_rows(hipStream_t stream, const void* a, int dtype, const float* ss, int pieces, int n_rows,
                             float eps, int width, void* out) {
    PALM_CHECK(n_rows >= 0 && width > 0 && pieces > 0, "scale_rows: rows=%d width=%d pieces=%d", n_rows, width, pieces);
    if (n_rows == 0) return 0;
    PALM_DTYPE_SWITCH(dtype, T,
        scale_rows_kernel<T><<<n_rows, 256, 0, stream>>>((const T*)a, ss, pieces, n_rows, eps, width, (T*)out));
    PALM_LAUNCHED();
    return 0;
}

// ---- SwiGLU ---------------------------------------------------------------------------------------
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int n_rows, int inter) {
    const size_t total = (size_t)n_rows * inter;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / inter, c = i % inter;
        const float g = to_float(gu[r * 2 * inter + c]);
        const float u = to_float(gu[r * 2 * inter + inter + c]);
        out[i] = from_float<T>(g / (1.0f + expf(-g)) * u);
    }
}

// bfloat16 rows whose half is a multiple of 8: eight outputs a thread, 16-byte reads and writes.  The library's expf
// and a full division are some thirty instructions an element, which made this pass wait for arithmetic rather than
// for memory (30.7 us for 2,048 x 12,288 outputs, 150 MB); the hardware's 2^x and reciprocal are one each and good to
// a unit in the last place of 32 bits, far below the rounding to bfloat16 that follows.  (The float32 mode takes
// swiglu_kernel above, with expf and the division.)
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ inline float silu_fast(float g) {
    return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * -1.4426950408889634f));
}
__global__ void swiglu_bf16x8_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out, int n_rows, int inter) {
    const int per_row = inter / 8;
    const size_t total = (size_t)n_rows * per_row;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / per_row, c = (i % per_row) * 8;
        const uint4 g4 = *reinterpret_cast<const uint4*>(gu + r * 2 * inter + c);
        const uint4 u4 = *reinterpret_cast<const uint4*>(gu + r * 2 * inter + inter + c);
        const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
        uint32_t ow[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float g0 = __uint_as_float(gw[j] << 16), g1 = __uint_as_float(gw[j] & 0xffff0000u);
            const float u0 = __uint_as_float(uw[j] << 16), u1 = __uint_as_float(uw[j] & 0xffff0000u);
            const bf16x2_t pair = {(__bf16)(silu_fast(g0) * u0), (__bf16)(silu_fast(g1) * u1)};      // round to nearest even
            ow[j] = __builtin_bit_cast(uint32_t, pair);
        }
        *reinterpret_cast<uint4*>(out + r * inter + c) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
    }
}

PALM_API int palm_swiglu(hipStream_t stream, const void* gate_up, int dtype, void* out, int n_rows, int inter) {
    PALM_CHECK(n_rows >= 0 && inter > 0, "swiglu: rows=%d intermediate=%d", n_rows, inter);
    if (n_rows == 0) return 0;
    if (dtype == PALM_BF16 && inter % 8 == 0 && ((uintptr_t)gate_up | (uintptr_t)out) % 16 == 0) {
        const size_t work = (size_t)n_rows * (inter / 8);
        const int blocks = (int)((work + 255) / 256 < 16384 ? (work + 255) / 256 : 16384);
        swiglu_bf16x8_kernel<<<blocks, 256, 0, stream>>>((const bf16_t*)gate_up, (bf16_t*)out, n_rows, inter);
        PALM_LAUNCHED();
        return 0;
    }
    const size_t total = (size_t)n_rows * inter;
    const int blocks = (int)((total + 255) / 256 < 65536 ? (total + 255) / 256 : 65536);
    PALM_DTYPE_SWITCH(dtype, T,
        swiglu_kernel<T><<<blocks, 256, 0, stream>>>((const T*)gate_up, (T*)out, n_rows, inter));
    PALM_LAUNCHED();
    return 0;
}

// y[r, c] += bias[c]: a projection's bias, added to the product in 32-bit and rounded once more to y's type.  The
// matrix-core kernels have no bias term in their epilogues (Qwen3's projections have none, models/qwen3.py:290-349);
// a part whose projection has one pays this pass.
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ y, const float* __restrict__ bias, size_t total, int cols) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x)
        y[i] = from_float<T>(to_float(y[i]) + bias[i % cols]);
}

PALM_API int palm_add_bias(hipStream_t stream, void* y, int dtype, const float* bias, int n_rows, int cols) {
    PALM_CHECK(n_rows >= 0 && cols > 0 && bias, "add_bias: rows=%d cols=%d", n_rows, cols);
    if (n_rows == 0) return 0;
    const size_t total = (size_t)n_rows * cols;
    const int blocks = (int)((total + 255) / 256 < 65536 ? (total + 255) / 256 : 65536);
    PALM_DTYPE_SWITCH(dtype, T, add_bias_kernel<T><<<blocks, 256, 0, stream>>>((T*)y, bias, total, cols));
    PALM_LAUNCHED();
    return 0;
}
