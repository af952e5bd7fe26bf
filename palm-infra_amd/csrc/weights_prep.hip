// What a model's parameters go through on their way into device memory: random numbers for the random-weights
// mode, and the conversion of a checkpoint tensor's stored type into the type the engine keeps, written into
// its rows of a (possibly joined) parameter.
//
// The reference converts and joins on the host when it packs a model (models/qwen3.py:125-160) and has random
// weights only as a numpy fixture (tests/run_tiny_qwen3_cpu_e2e.py:61-94).
//
// random_fill is counter-based: element i of a tensor is a function of (key, i) alone, where the key is made
// on the host from the seed and the tensor's name.  The same function is written in numpy in
// weights/random_numbers.py, and both give the same bits: every step below is one correctly rounded 32-bit
// operation (add, multiply, divide, square root) or integer arithmetic, in a fixed order, with no fused
// multiply-add (contraction is off for this file) and no library function.
//   h      = mix(key + (i + 1) * 0x9E3779B97F4A7C15)              (the splitmix64 finaliser)
//   u      = (2 * (h >> 41) + 1) / 2^24                           in (0, 1), exact
//   turn   = ((h >> 17) & 0xFFFFFF) / 2^24                        in [0, 1), exact
//   z      = sqrt(-2 ln u) * cos(2 pi turn)                       (Box-Muller)
//   value  = z * std + mean
// ln: u = m 2^e with m in (sqrt(1/2), sqrt(2)], ln m = 2 atanh((m-1)/(m+1)) as an odd series up to s^9.
// cos: the turn's top three bits name the octant, the rest an angle x in [0, pi/4) whose sine and cosine are
// series up to x^9 and x^8; the octant's identity combines them.
#include "common.h"

#pragma clang fp contract(off)

__host__ __device__ inline uint64_t mix64(uint64_t x) {
    x ^= x >> 30; x *= 0xBF58476D1CE4E5B9ull;
    x ^= x >> 27; x *= 0x94D049BB133111EBull;
    x ^= x >> 31;
    return x;
}

__device__ inline float normal_from_bits(uint64_t h) {
    const uint32_t a = (uint32_t)(h >> 41), b = (uint32_t)(h >> 17) & 0xFFFFFFu;
    const float u = (float)(2u * a + 1u) * 0x1p-24f;
    // ln u
    const uint32_t bits = __float_as_uint(u);
    int e = (int)(bits >> 23) - 127;
    float m = __uint_as_float((bits & 0x7FFFFFu) | 0x3F800000u);
    if (m > 0x1.6a09e6p+0f) { m = m * 0.5f; e += 1; }
    const float s = (m - 1.0f) / (m + 1.0f), s2 = s * s;
    float p = 0x1.c71c72p-4f;                  // 1/9
    p = p * s2 + 0x1.24924ap-3f;               // 1/7
    p = p * s2 + 0x1.99999ap-3f;               // 1/5
    p = p * s2 + 0x1.555556p-2f;               // 1/3
    p = p * s2 + 1.0f;
    const float ln_u = (float)e * 0x1.62e430p-1f + (s * p) * 2.0f;
    const float r = sqrtf(-2.0f * ln_u);
    // cos of the turn
    const uint32_t oct = b >> 21, f = b & 0x1FFFFFu;
    const float x = ((float)f * 0x1p-24f) * 0x1.921fb6p+2f, x2 = x * x;       // 2 pi
    float sp = 0x1.71de3ap-19f;                // 1/9!
    sp = sp * x2 + -0x1.a01a02p-13f;           // -1/7!
    sp = sp * x2 + 0x1.111112p-7f;             // 1/5!
    sp = sp * x2 + -0x1.555556p-3f;            // -1/3!
    sp = sp * x2 + 1.0f;
    const float sin_x = x * sp;
    float cp = 0x1.a01a02p-16f;                // 1/8!
    cp = cp * x2 + -0x1.6c16c2p-10f;           // -1/6!
    cp = cp * x2 + 0x1.555556p-5f;             // 1/4!
    cp = cp * x2 + -0.5f;
    cp = cp * x2 + 1.0f;
    const float cos_x = cp;
    const float half = 0x1.6a09e6p-1f;         // sqrt(1/2)
    const float diff = (cos_x - sin_x) * half, sum = (cos_x + sin_x) * half;
    float c;
    switch (oct) {
        case 0: c = cos_x; break;
        case 1: c = diff; break;
        case 2: c = -sin_x; break;
        case 3: c = -sum; break;
        case 4: c = -cos_x; break;
        case 5: c = -diff; break;
        case 6: c = sin_x; break;
        default: c = sum; break;
    }
    return r * c;
}

template <typename T>
__global__ void random_fill_kernel(T* __restrict__ out, size_t n, uint64_t key, float mean, float std) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const float z = normal_from_bits(mix64(key + (uint64_t)(i + 1) * 0x9E3779B97F4A7C15ull));
        out[i] = from_float<T>(z * std + mean);
    }
}

PALM_API int palm_random_fill(hipStream_t stream, void* out, int dtype, long long n, unsigned long long key, float mean,
                              float std) {
    PALM_CHECK(n >= 0 && out, "random_fill: n=%lld out=%p", n, out);
    if (n == 0) return 0;
    const int blocks = (int)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
    PALM_DTYPE_SWITCH(dtype, T, random_fill_kernel<T><<<blocks, 256, 0, stream>>>((T*)out, (size_t)n, (uint64_t)key, mean, std));
    PALM_LAUNCHED();
    return 0;
}

// ---- conversion at load ---------------------------------------------------------------------------
// Stored element types of a checkpoint's float tensors; the kept type is float32 or bfloat16 (codes 0 and 1).
enum StoredDtype : int { STORED_F32 = 0, STORED_BF16 = 1, STORED_F16 = 2, STORED_F64 = 3 };

__device__ inline float stored_to_float(float v) { return v; }
__device__ inline float stored_to_float(bf16_t v) { return to_float(v); }
__device__ inline float stored_to_float(_Float16 v) { return (float)v; }
__device__ inline float stored_to_float(double v) { return (float)v; }        // round to nearest

template <typename TS, typename TD>
__global__ void convert_kernel(const TS* __restrict__ src, TD* __restrict__ dst, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        dst[i] = from_float<TD>(stored_to_float(src[i]));
}

template <typename TS>
static int launch_convert(hipStream_t stream, const void* src, void* dst, int dst_dtype, size_t n) {
    const int blocks = (int)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
    PALM_DTYPE_SWITCH(dst_dtype, TD, convert_kernel<TS, TD><<<blocks, 256, 0, stream>>>((const TS*)src, (TD*)dst, n));
    PALM_LAUNCHED();
    return 0;
}

// dst[0 .. n) = src[0 .. n) in the kept type: one rounding to nearest (ties to even) where the kept type is
// narrower, exact where it is wider.  dst is usually a run of rows inside a joined parameter.
PALM_API int palm_convert(hipStream_t stream, const void* src, int stored_dtype, void* dst, int dst_dtype, long long n) {
    PALM_CHECK(n >= 0, "convert: n=%lld", n);
    if (n == 0) return 0;
    PALM_CHECK(src && dst, "convert: a null tensor");
    switch (stored_dtype) {
        case STORED_F32: return launch_convert<float>(stream, src, dst, dst_dtype, (size_t)n);
        case STORED_BF16: return launch_convert<bf16_t>(stream, src, dst, dst_dtype, (size_t)n);
        case STORED_F16: return launch_convert<_Float16>(stream, src, dst, dst_dtype, (size_t)n);
        case STORED_F64: return launch_convert<double>(stream, src, dst, dst_dtype, (size_t)n);
        default: return palm_fail("convert: stored type code %d is not float32 (0), bfloat16 (1), float16 (2) or float64 (3)", stored_dtype);
    }
}
