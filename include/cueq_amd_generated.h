/*
 * Entry points of the shared objects generated and compiled at first use for
 * one fully connected tensor product (cuequivariance_amd/codegen/fullyconnected.py,
 * loaded by cuequivariance_amd/jit.py).  The main library (cueq_amd.h) does not
 * export them: every generated object exports this same set, specialised for one
 * descriptor (its flattened paths, block shapes and coefficients are constants of
 * the code) and one element type (float, or bfloat16 passed as 16-bit words).
 *
 * They stand for the reference's fused dense operator with four operands,
 * FusedTensorProductOp4 (cuequivariance_torch/cuequivariance_torch/primitives/
 * segmented_polynomial_fused_tp.py:40-48, called at :228-262), in the form the
 * fully connected descriptor takes (descriptors/irreps_tp.py:22-91 with the second
 * operand of multiplicity one): weights W shared over the batch, x1 (Z x width_in),
 * x2 (Z x n2), out (Z x width_out), all row-major with a row stride in ELEMENTS.
 *
 * Every call launches asynchronously on `stream` (a hipStream_t), allocates
 * nothing, and returns 0, or -1 when the launch failed.  Rows are read and written
 * in 16-byte pieces: pointers and row strides of x1, out, g and dx1 must be
 * multiples of 16 bytes, and so must the pointer W (the weight blocks are brought
 * into the local data share in 16-byte pieces).
 */
#ifndef CUEQ_AMD_GENERATED_H
#define CUEQ_AMD_GENERATED_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* out[z, :] = sum over paths c * x2[z, j] * (x1[z, segment] @ W_block); writes every column of out */
int fcj_fwd(int64_t Z, const void* W, const void* x1, int64_t ld_x1, const void* x2, int64_t ld_x2, void* out, int64_t ld_out,
            void* stream);

/* dx1[z, :] for the cotangent g of out; writes every column of dx1 */
int fcj_dx1(int64_t Z, const void* W, const void* g, int64_t ld_g, const void* x2, int64_t ld_x2, void* dx1, int64_t ld_dx1,
            void* stream);

/* dx2[z, :]; writes every column of dx2 */
int fcj_dx2(int64_t Z, const void* W, const void* x1, int64_t ld_x1, const void* x2, int64_t ld_x2, const void* g, int64_t ld_g,
            void* dx2, int64_t ld_dx2, void* stream);

/* dx1 and dx2 from one pass over their common products g W^T (float objects whose multiplicities are multiples of 64;
 * every other object returns -2 and the caller uses fcj_dx1 and fcj_dx2).  part: 2 * (columns of x2) floats per row of
 * scratch that the caller provides; the two halves of every dx2 row are added in a fixed order (no atomics). */
int fcj_dx12(int64_t Z, const void* W, const void* g, int64_t ld_g, const void* x2, int64_t ld_x2, const void* x1, int64_t ld_x1,
             void* dx1, int64_t ld_dx1, void* dx2, int64_t ld_dx2, float* part, void* stream);

/* Weight gradient as per-block partial sums: fcj_dw writes part[b, 0 .. numel) (float, numel = number of weights) for
 * b < fcj_dw_blocks(Z); the caller provides part and sums its rows (cueq_sum_rows).  Weights no path touches are not
 * written: clear part first when the paths do not cover W. */
int fcj_dw_blocks(int64_t Z);
int fcj_dw(int64_t Z, const void* x1, int64_t ld_x1, const void* x2, int64_t ld_x2, const void* g, int64_t ld_g, float* part,
           int64_t numel, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* CUEQ_AMD_GENERATED_H */
