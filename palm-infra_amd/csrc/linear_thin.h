// What the kernels for products of up to 16 rows share: the epilogues' names, the step of K, and the norm that can be
// folded into a product.
#pragma once
#include "mfma.h"

enum ThinEpilogue : int { EPI_STORE = 0, EPI_SWIGLU = 1 };

constexpr int SUPER_K = 128;         // k-values of a "super-step": four matrix instructions of 32

// The norm around a product can be folded into it, which saves the norm's own kernel in a decode step.  RMSNorm is
// y = x * f * w with one factor f = 1 / sqrt(mean(x^2) + eps) for the row, so (x * f * w) . W^T = f * ((x * w) . W^T):
// a product whose activations are x * w, not yet multiplied by f, only has to multiply its result rows by f, and f
// needs nothing but the row's sum of squares.
//   out side: the product is a branch's output d.  The block that owns a strip of 16 features adds d to the
//             residual stream (x += d, each element by exactly one thread), stores x * w_out rounded to
//             bfloat16 as the next product's activations, and the strip's share of each row's sum of squares
//             in ss_out[row * strips + strip].
//   in side:  every block adds up the pieces ss_in[row * pieces + piece] in a fixed order, and multiplies its
//             results by f(row) before the epilogue.
struct RowNorm {
    const float* ss_in;      // [M, pieces_in] or null (a row's pieces side by side: 32 lanes read them in one go)
    int pieces_in;
    float eps_in;
    int width_in;            // the row length the mean is over
    float* resid;            // [M, N] float32, updated; or null
    const float* w_out;      // [N]
    float* ss_out;           // [M, strips]
};

// The stream of eight waves a block whose weights cross LDS (linear_ring.hip), for M <= 16 rows and K a multiple of 8.
// steps: super-steps a wave makes for one strip; parts: ranges of K (planes of the result).  A lane's place among its
// strip's rows, in the activations and in the residual stream is a 32-bit byte offset: 17 K and 16 N elements, which
// the entry point checks.
void launch_linear_ring(hipStream_t stream, const void* a, const void* w, void* c, int c_dtype, int M, int N, int K,
                        int epilogue, int parts, int steps, const RowNorm& norm);
