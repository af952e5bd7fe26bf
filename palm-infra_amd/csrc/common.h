// Shared pieces of the gfx950 kernels: element types, conversions, wave and block reductions, and
// the way entry points report a fault (a code and a message, never a silent wrong result).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <math.h>
#include <stdarg.h>

#define PALM_API extern "C" __attribute__((visibility("default")))

constexpr int WAVE = 64;          // lanes of a CDNA wavefront
constexpr int PAGE_TOKENS = 64;   // positions in one page of the key/value cache

// element type codes of the C interface
enum PalmDtype : int { PALM_F32 = 0, PALM_BF16 = 1 };

struct bf16_t { uint16_t bits; };

__host__ __device__ inline float to_float(float v) { return v; }
__host__ __device__ inline float to_float(bf16_t v) {
    union { uint32_t u; float f; } c;
    c.u = static_cast<uint32_t>(v.bits) << 16;
    return c.f;
}

// round to nearest, ties to even; NaN stays NaN.  On the device this is the hardware's conversion (one
// instruction for two values); the arithmetic below serves host code and says what the conversion does.
__host__ __device__ inline bf16_t f32_to_bf16(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
    bf16_t native;
    native.bits = __builtin_bit_cast(uint16_t, (__bf16)f);
    return native;
#endif
    union { uint32_t u; float f; } c;
    c.f = f;
    bf16_t r;
    if ((c.u & 0x7fffffffu) > 0x7f800000u) { r.bits = static_cast<uint16_t>((c.u >> 16) | 0x0040u); return r; }
    c.u += 0x7fffu + ((c.u >> 16) & 1u);
    r.bits = static_cast<uint16_t>(c.u >> 16);
    return r;
}

template <typename T> __host__ __device__ inline T from_float(float v);
template <> __host__ __device__ inline float from_float<float>(float v) { return v; }
template <> __host__ __device__ inline bf16_t from_float<bf16_t>(float v) { return f32_to_bf16(v); }

__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, WAVE);
    return v;
}
__device__ inline float wave_max(float v) {
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, WAVE));
    return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.  `scratch` holds 16 floats.
__device__ inline float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, n_waves = (blockDim.x + WAVE - 1) / WAVE;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < n_waves; ++w) total += scratch[w];
    return total;
}

// ---- errors -------------------------------------------------------------------------------------
// Entry points return 0 or a negative code; palm_last_error() gives the text of the last fault of
// the calling thread.
inline thread_local char g_palm_error[512] = "";
inline int palm_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_palm_error, sizeof(g_palm_error), fmt, ap);
    va_end(ap);
    return -1;
}
// Once in every shared library built from these sources:
#define PALM_DEFINE_LAST_ERROR() PALM_API const char* palm_last_error() { return g_palm_error; }
#define PALM_CHECK(cond, ...) do { if (!(cond)) return palm_fail(__VA_ARGS__); } while (0)
#define PALM_HIP(expr) do { hipError_t e_ = (expr); if (e_ != hipSuccess) \
    return palm_fail("%s failed: %s", #expr, hipGetErrorString(e_)); } while (0)
#define PALM_LAUNCHED() PALM_HIP(hipGetLastError())

// Dispatch on an element type code; `T` is the type inside the body.
#define PALM_DTYPE_SWITCH(code, T, ...) \
    switch (code) { \
        case PALM_F32: { using T = float; __VA_ARGS__; break; } \
        case PALM_BF16: { using T = bf16_t; __VA_ARGS__; break; } \
        default: return palm_fail("element type code %d is not float32 (0) or bfloat16 (1)", (int)(code)); \
    }
