// The entry points of the product for 17 to 128 rows (linear_wide.h has the kernel): the plan of a launch and the
// choice of the instance.
#include "linear_wide.h"

// Waves a block and ranges of K: what takes the fewest rounds of blocks over the compute units, a round
// costing its chunks (and two for its start) times the waves that share a unit's reads.
static int row_blocks_of(int M) { return M <= 32 ? 2 : (M <= 64 ? 4 : 8); }       // of 16 rows: the instance that serves M rows

static WidePlan wide_plan(int M, int N, int K, int epilogue, int max_parts) {
    const int strips = epilogue == WIDE_SWIGLU ? (N / 2 + 7) / 8 : (N + 15) / 16;
    const int chunk = wide_chunk(row_blocks_of(M));
    const int n_chunks = (K + chunk - 1) / chunk;
    WidePlan best{8, 1, n_chunks};
    long best_cost = -1;
    for (int parts = 1; parts <= max_parts; ++parts) {
        const int per = (n_chunks + parts - 1) / parts;
        if (parts > 1 && (per < WIDE_MIN_CHUNKS || (parts - 1) * per >= n_chunks)) continue;   // short, or an empty range
        for (int waves = 8; waves >= 4; waves -= 2) {       // of equals the larger block: it shares the rows among more strips
            const long blocks = (long)((strips + waves - 1) / waves) * parts;
            const long cost = ((blocks + WIDE_UNITS - 1) / WIDE_UNITS) * (per + 2) * waves;
            if (best_cost < 0 || cost < best_cost) { best_cost = cost; best = WidePlan{waves, parts, per}; }
        }
    }
    return best;
}

// Into how many planes the product comes if the caller takes planes (1: the result itself).
PALM_API int palm_linear_wide_parts(int M, int N, int K, int epilogue) {
    if (epilogue == WIDE_SWIGLU || N <= 0 || K <= 0) return 1;
    return wide_plan(M, N, K, epilogue, WIDE_MAX_PARTS).parts;
}

// How many blocks the launch would have: a caller with another way to the product takes that when these are few.
PALM_API int palm_linear_wide_blocks(int M, int N, int K, int epilogue, int planes_ok) {
    if (N <= 0 || K <= 0) return 0;
    const WidePlan plan = wide_plan(M, N, K, epilogue, planes_ok && epilogue == WIDE_STORE ? WIDE_MAX_PARTS : 1);
    const int strips = epilogue == WIDE_SWIGLU ? (N / 2 + 7) / 8 : (N + 15) / 16;
    return (strips + plan.waves - 1) / plan.waves * plan.parts;
}

// a [M, K] bfloat16 with M <= 128, w [N, K] bfloat16; c [M, N] (store) or [M, N/2] (gated) in bfloat16 or float32,
// or, with parts > 1 (as palm_linear_wide_parts says; store only), float32 planes [parts, M, N].
PALM_API int palm_linear_wide(hipStream_t stream, const void* a, const void* w, void* c, int c_dtype, int M, int N, int K,
                              int epilogue, int parts) {
    PALM_CHECK(M >= 0 && N > 0 && K > 0, "linear_wide: M=%d N=%d K=%d", M, N, K);
    PALM_CHECK(M <= WIDE_MAX_ROWS, "linear_wide: %d rows are more than the %d it shares through LDS", M, WIDE_MAX_ROWS);
    PALM_CHECK(K % 8 == 0, "linear_wide: K = %d is not a multiple of 8 (rows must start on 16 bytes)", K);
    PALM_CHECK(epilogue == WIDE_STORE || epilogue == WIDE_SWIGLU, "linear_wide: epilogue %d", epilogue);
    PALM_CHECK(epilogue != WIDE_SWIGLU || N % 2 == 0, "linear_wide: a gated product needs an even N, got %d", N);
    PALM_CHECK(((uintptr_t)a | (uintptr_t)w | (uintptr_t)c) % 16 == 0, "linear_wide: operands must be 16-byte aligned");
    PALM_CHECK(c_dtype == PALM_BF16 || c_dtype == PALM_F32, "linear_wide: result type %d", c_dtype);
    // a lane's place within its wave's rows, and a row's within the activations, are 32-bit byte offsets
    PALM_CHECK((double)(epilogue == WIDE_SWIGLU ? N / 2 + 8 : 16) * K * 2 < 4.0e9 && (double)WIDE_MAX_ROWS * K * 2 < 4.0e9,
               "linear_wide: N=%d K=%d is beyond 32-bit offsets", N, K);
    WidePlan plan = wide_plan(M, N, K, epilogue, parts > 1 ? WIDE_MAX_PARTS : 1);
    PALM_CHECK(parts == 1 || (parts == plan.parts && epilogue == WIDE_STORE && c_dtype == PALM_F32),
               "linear_wide: %d planes asked for, %d planned (planes are float32, not gated)", parts, plan.parts);
    if (M == 0) return 0;
    if (epilogue == WIDE_SWIGLU) {
        if (M <= 32) wide_launch_gated_32(stream, a, w, c, c_dtype, M, N, K, plan);
        else if (M <= 64) wide_launch_gated_64(stream, a, w, c, c_dtype, M, N, K, plan);
        else wide_launch_gated_128(stream, a, w, c, c_dtype, M, N, K, plan);
    } else {
        if (M <= 32) wide_launch_store_32(stream, a, w, c, c_dtype, M, N, K, plan);
        else if (M <= 64) wide_launch_store_64(stream, a, w, c, c_dtype, M, N, K, plan);
        else wide_launch_store_128(stream, a, w, c, c_dtype, M, N, K, plan);
    }
    PALM_LAUNCHED();
    return 0;
}
