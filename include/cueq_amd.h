/*
 * C ABI of the MI355X (gfx950) segmented-polynomial engine.
 *
 * Every entry point takes plain pointers and sizes, launches asynchronously on
 * the given HIP stream (passed as void*), never allocates device memory unless
 * stated, never throws, and returns 0 on success or a negative error code;
 * cueq_last_error() returns a thread-local message for the last failure.
 *
 * The entry points replace the closed native ops that the reference's Python
 * frontend calls; each declaration cites the reference call site it stands for
 * (paths relative to the reference checkout).
 */
#ifndef CUEQ_AMD_H
#define CUEQ_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types of tensors crossing the boundary */
enum cueq_dtype { CUEQ_F32 = 0, CUEQ_F64 = 1, CUEQ_F16 = 2, CUEQ_BF16 = 3 };

/* How a buffer's rows relate to the batch index z.
 * Mirrors BATCH_DIM_{AUTO,SHARED,BATCHED,INDEXED} imported at
 * cuequivariance_torch/cuequivariance_torch/primitives/segmented_polynomial_uniform_1d.py:25-30
 * (the reference does not publish the numeric values; these are this library's). */
enum cueq_batch_dim { CUEQ_BATCH_AUTO = -1, CUEQ_BATCH_SHARED = 0, CUEQ_BATCH_BATCHED = 1, CUEQ_BATCH_INDEXED = 2 };

enum cueq_status {
  CUEQ_OK = 0,
  CUEQ_ERR_INVALID = -1,     /* malformed tables / arguments                      */
  CUEQ_ERR_UNSUPPORTED = -2, /* valid request this build has no kernel for        */
  CUEQ_ERR_HIP = -3,         /* a HIP runtime call failed                         */
  CUEQ_ERR_TOO_LARGE = -4    /* size beyond a documented limit                    */
};

const char* cueq_last_error(void);
const char* cueq_version(void);

/* Process-wide options (no counterpart in the reference).  "deterministic": 1 makes the fused channel-wise backward
 * sum the gradient of a gathered operand in index order (bit-reproducible, one more pass) instead of scattering it
 * with floating-point atomics; "force_generic": 1 runs the table-driven kernels even where generated ones exist.
 * Initial values come from the environment variables CUEQ_DETERMINISTIC / CUEQ_FORCE_GENERIC ("1"), read once when
 * first needed.  cueq_get_option returns the value, or -1 for an unknown name. */
int cueq_set_option(const char* name, int32_t value);
int cueq_get_option(const char* name);

/* Per-kernel timing with HIP events recorded on the stream each kernel is launched on.
 * Between cueq_timing_begin() and cueq_timing_end() the main kernel of every call is bracketed by a
 * pair of events; cueq_timing_end waits for them and returns, per kernel name, the number of launches
 * and their summed duration.  Same purpose as the reference's event-based helper
 * cuequivariance_torch/cuequivariance_torch/benchmarking.py:24-158; unlike it, the events sit directly
 * around the kernel inside the library, so host-side launch work is excluded. */
/* Memory-system calibration (no counterpart in the reference): one launch of a streaming kernel shaped like the
 * path-table kernels (64-thread workgroups, a dword per lane and instruction, 8 wavefronts per compute unit) over
 * `bytes` of the two device buffers; kind 0 reads `in`, 1 writes `out`, 2 adds to `out` with float atomics, 3 copies.
 * Time it with cueq_timing_begin / cueq_timing_end (labels calibrate_read / _write / _atomic / _copy). */
int cueq_calibrate(int32_t kind, const void* in, void* out, int64_t bytes, void* stream);

typedef struct {
  char name[64];
  int64_t launches;
  double total_ms;
} cueq_timing_entry;
int cueq_timing_begin(void);
int cueq_timing_end(cueq_timing_entry* entries, int max_entries); /* returns the number of entries filled */

/* ------------------------------------------------------------------------- */
/* uniform-1d executor                                                        */
/* ------------------------------------------------------------------------- */

typedef struct cueq_u1d_plan cueq_u1d_plan;

/* Descriptor tables, exactly the flat lists the reference builds at
 * cuequivariance_torch/cuequivariance_torch/primitives/segmented_polynomial_uniform_1d.py:188-218
 * and passes positionally to torch.ops.cuequivariance.uniform_1d (same file, :55-77). */
typedef struct {
  int32_t math_dtype;                  /* CUEQ_F32 or CUEQ_F64                                   */
  int64_t operand_extent;              /* u: extent of the single mode                            */
  int32_t num_inputs;
  int32_t num_outputs;
  const int32_t* buffer_dim;           /* [num_inputs+num_outputs] 0: scalar segments, 1: u-vectors */
  const int32_t* buffer_num_segments;  /* [num_inputs+num_outputs]                                */
  int32_t num_operations;
  const int32_t* num_operands;         /* [num_operations]                                        */
  const int32_t* operations;           /* concatenated buffer ids, sum(num_operands) entries      */
  const int32_t* num_paths;            /* [num_operations]                                        */
  const int64_t* path_indices_start;   /* [num_operations] offset into path_indices               */
  const int64_t* path_coefficients_start; /* [num_operations] offset into path_coefficients      */
  const int32_t* path_indices;         /* row-major (path, operand) segment ids                   */
  int64_t path_indices_len;
  const double* path_coefficients;
  int64_t path_coefficients_len;
  /* Optional row layouts (no counterpart in the reference's tables, where a transposition module sits in front of the op:
   * cuequivariance_torch/cuequivariance_torch/primitives/transpose.py:83-183).  Default (both NULL, or 0 groups for a
   * buffer): segment s, channel u at s * extent + u ("ir_mul").  With groups (d_0, d_1, ...) partitioning the segments of
   * a channel-carrying buffer, the rows are stored group by group, channel-major inside a group ("mul_ir"): segment c of
   * group g, channel u at extent * (d_0 + ... + d_{g-1}) + u * d_g + c.  The kernels address such rows directly. */
  const int32_t* layout_num_groups;    /* [num_inputs+num_outputs] or NULL                          */
  const int32_t* layout_group_dims;    /* the group sizes of all buffers, concatenated              */
} cueq_u1d_desc;

/* One tensor at the boundary. */
typedef struct {
  void* data;            /* device pointer, row-major (rows, num_segments * (dim ? extent : 1))   */
  int64_t rows;
  int32_t dtype;         /* cueq_dtype                                                            */
  int32_t batch_dim;     /* cueq_batch_dim (never AUTO here)                                      */
  const void* index;     /* INDEXED: device pointer to batch_size row ids, else NULL              */
  int32_t index_is_64;   /* 1: int64 ids, 0: int32                                                */
  /* Outputs that are INDEXED or SHARED are reduced without atomics.  For INDEXED the
   * caller passes the grouping of batch rows by output row: csr_offsets[rows+1] and
   * csr_perm[batch_size] (batch ids of row r are csr_perm[csr_offsets[r] .. csr_offsets[r+1]),
   * ascending inside a row), e.g. from cueq_segment_csr_build.  NULL otherwise.              */
  const int64_t* csr_offsets;
  const int64_t* csr_perm;
} cueq_u1d_buffer;

/* Compiles the tables into device-resident path tables (sorted and grouped by output
 * segment).  Allocates device memory owned by the plan.  The plan is immutable and may be
 * run concurrently from several threads/streams of the device it was created on. */
int cueq_u1d_plan_create(const cueq_u1d_desc* desc, cueq_u1d_plan** plan);
void cueq_u1d_plan_destroy(cueq_u1d_plan* plan);

/* Introspection: returns 1 when kernels specialised for this descriptor were compiled into the
 * library (0: the table-driven kernels will run); *hash receives the descriptor's content hash.
 * No counterpart in the reference, whose op compiles its kernel at run time
 * (CHANGELOG.md:38 "NVRTC"); here specialisation happens when the library is built. */
int cueq_u1d_plan_info(const cueq_u1d_plan* plan, uint64_t* hash);
/* Same answer from the tables alone; touches no device (usable on a host without a GPU). */
int cueq_u1d_desc_info(const cueq_u1d_desc* desc, uint64_t* hash);
/* The same question for buffers of one element type (a CUEQ_* code): the specialised kernels of a descriptor exist per
 * element type of the buffers - the arithmetic type itself (what cueq_u1d_desc_info reports) and, for float arithmetic,
 * bfloat16 and half (loaded and stored as 16-bit elements, computed in float: the reference's math_dtype=float32 with
 * 16-bit tensors, cuequivariance_torch/primitives/segmented_polynomial_uniform_1d.py:254-260).  Host-only. */
int cueq_u1d_desc_serves(const cueq_u1d_desc* desc, int32_t io_dtype);

/* Bytes of device workspace cueq_u1d_run needs for this call shape (0 if none). */
int64_t cueq_u1d_workspace_size(const cueq_u1d_plan* plan, const cueq_u1d_buffer* buffers, int64_t batch_size);

/* Evaluates every operation of the plan:
 *   out[b_out][row_out(z), seg_out(p), :] += coeff[p] * prod_k in[b_k][row_k(z), seg_k(p), :]
 * buffers = inputs then outputs; outputs are fully overwritten.  Stands for the call at
 * cuequivariance_torch/cuequivariance_torch/primitives/segmented_polynomial_uniform_1d.py:294-316. */
int cueq_u1d_run(const cueq_u1d_plan* plan, const cueq_u1d_buffer* buffers, int64_t batch_size,
                 void* workspace, int64_t workspace_bytes, void* stream);

/* cueq_u1d_run for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and results as cueq_u1d_run,
 * but the workspace is a static device array of cueq_u1d_static_scratch_bytes() (32 MiB) that every device running
 * the library holds until the process ends; the call allocates nothing.  A call shape whose
 * cueq_u1d_workspace_size exceeds that returns CUEQ_ERR_TOO_LARGE.  All calls on one device share the array:
 * calls that overlap on one device (different streams or threads) race; calls on one stream do not.  The first call on a
 * device looks the array's address up (a host-side query, not a stream operation): make one call on each device before
 * recording the entry point into a HIP graph. */
int64_t cueq_u1d_static_scratch_bytes(void);
int cueq_u1d_run_static(const cueq_u1d_plan* plan, const cueq_u1d_buffer* buffers, int64_t batch_size, void* stream);

/* Stable grouping of n row ids (values in [0, nrows)) by value: offsets[nrows+1], perm[n].
 * Deterministic (no atomics decide the order).  workspace: cueq_segment_csr_workspace(n, nrows) bytes. */
int64_t cueq_segment_csr_workspace(int64_t n, int64_t nrows);
int cueq_segment_csr_build(const void* index, int32_t index_is_64, int64_t n, int64_t nrows,
                           int64_t* offsets, int64_t* perm, void* workspace, int64_t workspace_bytes, void* stream);
/* Same grouping with device-side work only (always sorts; no host synchronisation, no memset node), so it can be
 * recorded into a HIP graph and regroups from the live index buffer at every replay.  cueq_segment_csr_build reads two
 * flags on the host (ids sorted already? in range?) and therefore cannot be captured.  Ids outside [0, nrows) cannot
 * be reported here: they are left out of every row.  Same workspace size. */
int cueq_segment_csr_build_async(const void* index, int32_t index_is_64, int64_t n, int64_t nrows,
                                 int64_t* offsets, int64_t* perm, void* workspace, int64_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------- */
/* dense segmented contractions (matrix cores)                                */
/* ------------------------------------------------------------------------- */

/* One small GEMM of a flattened Linear / fully-connected polynomial:
 *   C[z, c_off : c_off+N] (+)= alpha * S[z, s_col] * A[z, a_off : a_off+K] @ W,   W = K x N block of B at b_off
 * (trans_b: the block is stored N x K).  Replaces the closed modules FusedTensorProductOp3 / Op4 constructed at
 * cuequivariance_torch/cuequivariance_torch/primitives/segmented_polynomial_fused_tp.py:27-72. */
typedef struct {
  int64_t a_off, c_off, b_off;
  double alpha;
  int32_t s_col;      /* column of the per-row scalar in S, -1: none */
  int32_t trans_b;
  int32_t accumulate; /* 0: overwrite the output segment, 1: add to it */
  int32_t reserved;
} cueq_gemm_problem;

/* `problems` is a DEVICE pointer to nproblems entries (uploaded once by the caller when the layer is built; the
 * kernels read it with scalar loads).  All problems of one call share K, N, the row strides lda/lds/ldc (in
 * elements, lda a multiple of 8, every a_off a multiple of 8 for the MFMA kernels) and must write disjoint output
 * segments.  dtype: CUEQ_F32 / CUEQ_BF16 run on MFMA when K, N are in {32, 64, 128} and force_simple is 0;
 * otherwise, and for CUEQ_F64, a plain kernel runs.  Accumulation is in fp32 (fp64 for CUEQ_F64). */
int cueq_seg_gemm(int32_t dtype, int32_t K, int32_t N, const void* A, int64_t lda, const void* B, const void* S,
                  int64_t lds, void* C, int64_t ldc, int64_t rows, const cueq_gemm_problem* problems, int32_t nproblems,
                  int32_t force_simple, void* stream);

/* Weight gradient of the same contraction, summed over the batch without atomics:
 *   dW[k][n] (+)= sum_e sum_z alpha_e * S[z, s_col_e] * A[z, a_off_e + k] * G[z, c_off_e + n]
 * (trans_out: dW stored N x K).  `entries` is a DEVICE pointer.  workspace: cueq_seg_outer_workspace bytes. */
typedef struct {
  int64_t a_off, c_off;
  double alpha;
  int32_t s_col;
  int32_t reserved;
} cueq_outer_entry;
int64_t cueq_seg_outer_workspace(int32_t dtype, int32_t K, int32_t N, int64_t rows);
int cueq_seg_outer(int32_t dtype, int32_t K, int32_t N, const void* A, int64_t lda, const void* G, int64_t ldg,
                   const void* S, int64_t lds, void* dW, int64_t rows, const cueq_outer_entry* entries, int32_t nentries,
                   int32_t trans_out, int32_t accumulate, void* workspace, int64_t workspace_bytes, void* stream);

/* Gradient of the per-row scalar:  dS[z, s_col] (+)= alpha * sum_n G[z, c_off + n] * (A[z, a_off : a_off+K] @ W)[n]. */
int cueq_seg_rowdot(int32_t dtype, int32_t K, int32_t N, const void* A, int64_t lda, const void* B, const void* G,
                    int64_t ldg, void* dS, int64_t lds, int64_t rows, const cueq_gemm_problem* problem, void* stream);

/* Element-wise stages of the fully-connected product (uvw,iu,jv,kw with v = 1; FusedTensorProductOp4,
 * primitives/segmented_polynomial_fused_tp.py:40-48) on top of the tiled GEMMs: with T[:, t] = x1[:, i_seg] . W_p from cueq_gemm,
 *   cueq_fc_combine: O[z, out_off + n] = sum over the uses u of block b of coeff_u * S[z, j_u] * T[z, src_off_u + n],  n < n_b
 *   cueq_fc_rowdot:  D[z, j] = sum over the uses u with j_u == j of coeff_u * <X[z, a_off_u : +k_u], G[z, g_off_u : +k_u]>
 * blocks: device array of {int32 out_off, n, first_use, num_uses}; uses: device array of {int32 j, src_off; float coeff; int32 pad}
 * (combine) or {int32 j, a_off, g_off, k; float coeff; int32 pad[3]} (rowdot).  dtype: S, O, X, D (float32 / bfloat16);
 * t_dtype / g_dtype: T / G (float32 or the same).  Block widths at most max_n <= 256; D has n2 <= 64 columns.
 * vectorised != 0: the caller states that every block width, out_off and src_off in the tables is a multiple of four
 * (rowdot: every k, a_off and g_off) (then, with matching row strides and pointers, a thread moves four adjacent
 * elements at a time). */
int cueq_fc_combine(int32_t dtype, int32_t t_dtype, int64_t rows, const void* S, int64_t lds, const void* T, int64_t ldt, void* O,
                    int64_t ldo, const void* blocks, int32_t num_blocks, const void* uses, int32_t max_n, int32_t vectorised,
                    void* stream);
int cueq_fc_rowdot(int32_t dtype, int32_t g_dtype, int64_t rows, const void* X, int64_t ldx, const void* G, int64_t ldg, void* D,
                   int64_t ldd, int32_t n2, const void* uses, int32_t num_uses, int32_t vectorised, void* stream);

/* Element-wise stage of the fully connected contraction with a second operand of any multiplicity (form u_v_uvw_w of
 * FusedTensorProductOp4, primitives/segmented_polynomial_fused_tp.py:40-48, list of forms :114-129): the row-wise outer
 * products of operand segments, which a Linear map (cueq_gemm_table / cueq_gemm_nt) then contracts with the weights read as
 * (u v) x w matrices, and the two contractions that are its gradients.  parts: device array of nparts records
 * {int32 a_off, b_off, p_off, na, nb} (element offsets inside a row of A, B, P; extents of the two segments).
 *   cueq_outer_rows:           P[z, p_off + u * nb + v] = A[z, a_off + u] * B[z, b_off + v]   (a_major != 0)
 *                              P[z, p_off + v * na + u] = the same product                    (a_major == 0)
 *   cueq_outer_rows_contract:  which == 0:  O[z, a_off + u] = sum over the parts p of the segment and v of P[z, ..] * X[z, b_off_p + v]
 *                              which == 1:  O[z, b_off + v] = sum over the parts p of the segment and u of P[z, ..] * X[z, a_off_p + u]
 * Segments (of A for which == 0, of B for which == 1): seg_start (device, nsegs + 1 entries) delimits, in seg_parts (device),
 * the parts that read the segment; they are added in that order.  Columns of O outside the listed segments are not written.
 * max_part: the largest na * nb; max_extent: the largest extent of a listed segment (they size the grids).  Row strides in
 * elements; a row stride of 0 reads one row for every z.  dtype (all tensors): float64, float32, or bfloat16 / half with
 * products and sums in float32, rounded once.
 * vectorised = 4 or 8: the caller states that every offset and every extent of the fast index of P (nb if a_major, else na) in
 * the table is a multiple of that number (then, with matching row strides and pointers, a thread moves four adjacent elements
 * at a time, eight of a 2-byte type); 0: no such statement.  The three operations are closed under differentiation: the gradients of each are the other two. */
int cueq_outer_rows(int32_t dtype, int64_t rows, const void* A, int64_t lda, const void* B, int64_t ldb, void* P, int64_t ldp,
                    const void* parts, int32_t nparts, int32_t max_part, int32_t a_major, int32_t vectorised, void* stream);
int cueq_outer_rows_contract(int32_t dtype, int32_t which, int64_t rows, const void* Q, int64_t ldq, const void* X, int64_t ldx, void* O,
                             int64_t ldo, const void* parts, const int32_t* seg_start, const int32_t* seg_parts, int32_t nsegs,
                             int32_t max_extent, int32_t a_major, int32_t vectorised, void* stream);

/* ------------------------------------------------------------------------- */
/* triangle multiplicative update: the stages behind                           */
/*   cuequivariance_torch/cuequivariance_torch/primitives/triangle.py:138-262   */
/* (closed kernel; open algorithm cuequivariance_jax/cuequivariance_jax/triangle/  */
/*  _triangle_multiplicative_update.py:371-417).  dtype arguments are CUEQ_F32 or  */
/* CUEQ_BF16, arithmetic is fp32, all pointers are device pointers.                */
/* ------------------------------------------------------------------------- */

/* Batched C[b] = alpha * A[b] * B[b]^T (+ C[b]):  A is M x K (row stride lda), B is N x K (row stride ldb), both with the
 * contraction index contiguous; C is M x N (row stride ldc); strides between batch items in elements.  MFMA path when
 * K, lda, ldb and the batch strides are multiples of 16 bytes worth of elements, otherwise a plain kernel.
 * Stands for the projections (_sigmoid_gated_dual_gemm.py:111-150) and the contraction
 * einsum("dbik,dbjk->dbij") (_triangle_multiplicative_update.py:393-397). */
int cueq_gemm_nt(int32_t in_dtype, int32_t out_dtype, int64_t M, int64_t N, int64_t K, const void* A, int64_t lda,
                 int64_t stride_a, const void* B, int64_t ldb, int64_t stride_b, void* C, int64_t ldc, int64_t stride_c,
                 int64_t batch, double alpha, int32_t accumulate, void* stream);

/* cueq_gemm_nt with a choice of operand order: trans_a != 0 takes A as K x M (row stride lda, batch stride stride_a)
 * instead of M x K, trans_b != 0 takes B as K x N.  Serves the gradients of the triangular contraction
 * (da = dt b, db = dt^T a; _triangle_multiplicative_update.py:393-397) and its "incoming" form without transposed
 * copies.  Mixed input / output types are supported for trans_a == trans_b == 0 only.
 * Sizes: M, N, K below 2^31; one launch takes 8 355 840 rows (its row tiles sit on grid.y) and 65 535 batch items
 * (grid.z): more run as consecutive launches over slabs of rows / batch items (rows also in cueq_gemm_table and
 * cueq_dual_gate). */
int cueq_gemm(int32_t in_dtype, int32_t out_dtype, int32_t trans_a, int32_t trans_b, int64_t M, int64_t N, int64_t K,
              const void* A, int64_t lda, int64_t stride_a, const void* B, int64_t ldb, int64_t stride_b, void* C, int64_t ldc,
              int64_t stride_c, int64_t batch, double alpha, int32_t accumulate, void* stream);

/* The tiled product over unrelated blocks in one launch: part p computes C + table[3p+2] (+)= alpha * op(A + table[3p]) .
 * op(B + table[3p+1])^T with the shared extents M, N, K and row strides (table: device, int64, element offsets).
 * k_chunks > 1 (trans_a and trans_b only) cuts the contraction into k_chunks row ranges; chunk c writes its partial
 * product to C + c * chunk_stride_c + table[3p+2] and the caller adds the chunks in order.  Serves the weight contractions
 * of the fully-connected product (FusedTensorProductOp4, primitives/segmented_polynomial_fused_tp.py:40-48), whose blocks
 * do not advance by constant strides. */
int cueq_gemm_table(int32_t in_dtype, int32_t out_dtype, int32_t trans_a, int32_t trans_b, int64_t M, int64_t N, int64_t K,
                    const void* A, int64_t lda, const void* B, int64_t ldb, void* C, int64_t ldc, const int64_t* table,
                    int64_t nparts, int64_t k_chunks, int64_t chunk_stride_c, double alpha, int32_t accumulate, void* stream);

/* Row-streaming form of the same product, meant for the forward and the input gradient of Linear
 * (descriptor uv,iu,iv per irrep; FusedTensorProductOp3, primitives/segmented_polynomial_fused_tp.py:40-48):
 *   C[z, c_p : c_p + N] = alpha * A[z, a_p : a_p + K] . W_p      for all rows z < M and the parts p of the table,
 * where W_p = W + w_p is K x N as it lies (w_contraction_major != 0) or N x K (w_contraction_major == 0).  table: HOST
 * memory, nparts rows of (a_p, w_p, c_p) in elements, multiples of 16 bytes, inside a row resp. the w_numel elements of W;
 * the parts must write disjoint columns.  dtype: bfloat16 or float32 (A, W and C alike; float32 accumulation).
 * All distinct weight blocks of the launch stay in the local data share: K, N in {32, 64, 96, 128}, at most 8 distinct
 * blocks and 48 parts, (blocks * N * (K * element size + 16) + 36 864) bytes <= 160 KiB, else CUEQ_ERR_TOO_LARGE /
 * CUEQ_ERR_UNSUPPORTED (the caller then splits the parts over several launches or takes cueq_gemm_table). */
int cueq_linear_rows(int32_t dtype, int32_t w_contraction_major, int64_t M, int64_t N, int64_t K, const void* A, int64_t lda,
                     const void* W, int64_t w_numel, void* C, int64_t ldc, const int64_t* table, int64_t nparts, double alpha, void* stream);

/* The same launch for rows that keep the irrep component contiguous (`mul_ir`: element (channel u, component i) of a block
 * of D components at u * D + i).  The reference converts such rows to channel-contiguous ones in front of its dense
 * kernels and back behind them (cuequivariance_torch/primitives/transpose.py:83-183, called from
 * operations/linear.py:153-191); this entry point reads and writes them as they lie:
 *   C[z, c_p + v * D_p + i] = alpha * sum_u A[z, a_p + u * D_p + i] * W_p[u, v]     for i < D_p, all rows z < M and parts p.
 * table: HOST memory, nparts rows of (a_p, w_p, c_p, D_p); part p reads K * D_p and writes N * D_p consecutive elements of a
 * row; D_p in {1, 3, 5, 7}, mixed freely in one launch (all blocks of a row in one launch is also what the memory system
 * likes best).  N in {32, 64, 96, 128}; K a multiple of 64 (bfloat16) or 32 (float32) up to 128; other limits as for
 * cueq_linear_rows, with (blocks * N * (K * element size + 16) + waves * 16 * (128 * Dmax + 16)) bytes <= 160 KiB,
 * Dmax = max(3, largest D_p), waves = 8 if Dmax * N <= 384 else 4. */
int cueq_linear_rows_mul_ir(int32_t dtype, int32_t w_contraction_major, int64_t M, int64_t N, int64_t K, const void* A, int64_t lda,
                            const void* W, int64_t w_numel, void* C, int64_t ldc, const int64_t* table, int64_t nparts, double alpha,
                            void* stream);

/* Weight gradient of the same operation on `mul_ir` rows (the reference reaches it through autograd of its dense kernel
 * after the transposition of cuequivariance_torch/primitives/transpose.py:83-183):
 *   dW_p[u, v] = alpha * sum_{z < rows} sum_{i < D_p} A[z, a_p + u * D_p + i] * G[z, c_p + v * D_p + i]     (K x N, row-major)
 * table: HOST memory, nparts (<= 32) rows of (a_p, c_p, D_p), D_p in {1, 3, 5, 7}, offsets multiples of 16 bytes; K, N in
 * {32, 64, 96, 128}; bfloat16 or float32 inputs, float32 partial results.  Part p is cut into chunks of rows (counts in
 * proportion to 2 D_p + 1); chunk c of part p writes its partial product to row first_item[p] + c of `partials` (K * N floats per
 * row), and the caller adds the rows first_item[p] .. first_item[p + 1] - 1 in order (cueq_sum_rows): no atomics.
 * cueq_linear_dw_mul_ir_items returns the number of rows `partials` needs for this call shape on the current device and
 * fills first_item (nparts + 1 entries; may be NULL); -1 for a bad argument. */
int64_t cueq_linear_dw_mul_ir_items(int64_t rows, const int64_t* table, int32_t nparts, int32_t* first_item);
int cueq_linear_dw_mul_ir(int32_t dtype, int64_t K, int64_t N, int64_t rows, const void* A, int64_t lda, const void* G, int64_t ldg,
                          const int64_t* table, int32_t nparts, float* partials, double alpha, void* stream);

/* Grouped products on the tiled kernel, for a Linear whose weights are chosen per row by a sorted class index
 * (the closed indexed_linear op behind cuequivariance_torch/primitives/segmented_polynomial_indexed_linear.py:116-156):
 * offsets (device, int64, ngroups + 1) gives the row range [offsets[g], offsets[g+1]) of group g.
 *   mode 1, rows grouped:        C[z, :] (+)= alpha * A[z, :K] . B_g^T for the rows z of group g, B_g = B + g * group_stride
 *                                (N x K, or K x N with trans_b); batch items advance A, B, C by stride_* (column blocks).
 *   mode 2, contraction grouped: C_g (M x N at C + g * group_stride) (+)= alpha * sum over the rows z of group g of
 *                                A[z, :M]^T B[z, :N]; K is ignored; out_dtype may be float32 for bfloat16 inputs.
 * Extents along vectors, strides and pointers must be multiples of 16 bytes (CUEQ_ERR_UNSUPPORTED otherwise). */
int cueq_gemm_grouped(int32_t in_dtype, int32_t out_dtype, int32_t mode, int64_t M, int64_t N, int64_t K, const void* A, int64_t lda,
                      int64_t stride_a, const void* B, int64_t ldb, int64_t stride_b, void* C, int64_t ldc, int64_t stride_c,
                      int64_t batch, const int64_t* offsets, int64_t ngroups, int32_t trans_b, int64_t group_stride, double alpha,
                      int32_t accumulate, void* stream);

/* The gated dual projection in one kernel (_sigmoid_gated_dual_gemm.py:111-218): u = A1 B1^T, v = A2 B2^T (A* M x K, B* N x K,
 * contraction contiguous; B2 NULL: same as B1), then
 *   backward == 0:  out1 = sigmoid(u + bias1) * (v + bias2) * mask
 *   backward != 0:  out1 = d u, out2 = d v from the cotangent dC of that output (u, v are recomputed, never stored).
 * Biases / mask (may be NULL) are indexed by the row (axis 0) or column (axis 1) of the M x N result; ldc is the row
 * stride of dC, out1, out2.  K, lda, ldb and the operand pointers must be multiples of 16 bytes. */
int cueq_dual_gate(int32_t dtype, int32_t backward, int64_t M, int64_t N, int64_t K, const void* A1, const void* A2, int64_t lda,
                   const void* B1, const void* B2, int64_t ldb, const void* bias1, const void* bias2, int32_t bias_axis,
                   const void* mask, int32_t mask_axis, const void* dC, void* out1, void* out2, int64_t ldc, void* stream);

/* LayerNorm of the rows of X followed by the gated dual projection with the weights as rows, in one kernel - the first two
 * stages of the triangle update (cuequivariance_jax/cuequivariance_jax/triangle/_triangle_multiplicative_update.py:371-400:
 * x_hat = LN(x), then sigmoid(x_hat G^T + b) * (x_hat P^T + b) * mask written "transposed"):
 *   xhat[m, :] = (X[m, :] - mean[m]) * rstd[m] * gamma + beta   (biased variance, rstd = 1 / sqrt(var + eps); gamma / beta may be NULL)
 *   out[c, m]  = sigmoid(W1[c, :] . xhat[m, :] + bias1[c]) * (W2[c, :] . xhat[m, :] + bias2[c]) * mask[m]
 * with xhat rounded to bfloat16 before the products, as a separate cueq_layer_norm_fwd would have stored it; xhat (M x K, row
 * stride ldxh), mean and rstd (M floats each) are written for the later stages.  bfloat16 only, K = 32, 64, 96 or 128, C a
 * multiple of 32 with both weight matrices fitting the local data share, M even and at least 4096, ldc even; other shapes
 * return CUEQ_ERR_UNSUPPORTED (compose cueq_layer_norm_fwd and cueq_dual_gate instead). */
int cueq_ln_dual_gate(int32_t dtype, int64_t C, int64_t M, int64_t K, const void* W1, const void* W2, int64_t ldw, const void* X,
                      int64_t ldx, const void* gamma, const void* beta, double eps, const void* bias1, const void* bias2,
                      const void* mask, void* out, int64_t ldc, void* xhat, int64_t ldxh, float* mean, float* rstd, void* stream);

/* Backward of the gated dual projection down to the projection inputs (_sigmoid_gated_dual_gemm.py:153-218), one kernel:
 *   u[c][m] = W1[c,:] . X1[m,:],  v[c][m] = W2[c,:] . X2[m,:]   (W* C x K row-major with row stride ldw, X* M x K; recomputed)
 *   s = sigmoid(u + bias1[c]),  d = dC * mask[m],  du = d (v + bias2[c]) s (1 - s),  dv = d s
 *   X2 NULL or == X1:  dX1[m,:] (+)= sum_c du W1[c,:] + dv W2[c,:]          (accumulate != 0 adds to dX1)
 *   otherwise:         dX1[m,:]  =  sum_c du W1[c,:],   dX2[m,:] = sum_c dv W2[c,:]
 * dC (and dU, dV when not NULL: the gate gradients for the weight / bias gradients) are C x M with row stride ldc when
 * dc_by_row != 0, M x C otherwise (built for one input with dC by rows and for two inputs with dC by columns).
 * K must be 32, 64, 96 or 128 and C a multiple of 32; strides and pointers multiples of 16 bytes, else
 * CUEQ_ERR_UNSUPPORTED (compose cueq_dual_gate and cueq_gemm_nt instead).  dC by columns is addressed with 32-bit byte
 * offsets inside a launch: beyond 4 GiB of dC the rows run as consecutive launches over slabs of rows. */
int cueq_gate_bwd_input(int32_t dtype, int64_t C, int64_t M, int64_t K, const void* W1, const void* W2, int64_t ldw,
                        const void* X1, const void* X2, int64_t ldx,
                        const void* bias1, const void* bias2, const void* mask, const void* dC, int64_t ldc,
                        int32_t dc_by_row, void* dX1, void* dX2, int64_t lddx, int32_t accumulate, void* dU, void* dV,
                        void* stream);

/* cueq_gate_bwd_input in its one-input form with dC by rows, continued through the LayerNorm that produced X
 * (cuequivariance_jax/cuequivariance_jax/triangle/_triangle_multiplicative_update.py:371-400 backwards: the gradient of the input
 * projections and of x_hat = LN(x) in one kernel): with d = (dX if accumulate else 0) + sum_c du[c][m] W1[c,:] + dv[c][m] W2[c,:],
 *   g = d * ln_gamma,  xn = (ln_x - ln_mean) * ln_rstd,  dX[m,:] = ln_rstd[m] * (g - mean_k(g) - xn * mean_k(g * xn))
 * (ln_x: the M x K rows the LayerNorm took, row stride ldlx; ln_gamma may be NULL).  The gradients of gamma / beta and the gate
 * gradients are not formed here.  bfloat16 only, same shape limits as the resident form of cueq_gate_bwd_input; otherwise
 * CUEQ_ERR_UNSUPPORTED (compose cueq_gate_bwd_input and cueq_layer_norm_bwd instead). */
int cueq_gate_bwd_input_ln(int32_t dtype, int64_t C, int64_t M, int64_t K, const void* W1, const void* W2, int64_t ldw, const void* X,
                           int64_t ldx, const void* bias1, const void* bias2, const void* mask, const void* dC, int64_t ldc, void* dX,
                           int64_t lddx, int32_t accumulate, const void* ln_x, int64_t ldlx, const float* ln_mean, const float* ln_rstd,
                           const void* ln_gamma, void* stream);

/* Weight-gradient shaped product C (M x N) = sum over rows z and parts p of A[z, p*stride_a : +M]^T B[z, p*stride_b : +N]
 * (both operands row-major with the long index z as rows).  The rows are cut into chunks = items / nparts pieces; item
 * (part, chunk) writes alpha * its partial product to partials[part * chunks + chunk] (float32, M x N): the partials of one
 * part are consecutive, so the caller adds all cueq_gemm_tn_items(rows, nparts) items in order (cueq_sum_rows over an
 * items x (M*N) view) or, for parts that belong to different results, each run of parts on its own: no atomics.  Serves the weight gradients of the dense
 * layers (reference: the backward of FusedTensorProductOp3, primitives/segmented_polynomial_fused_tp.py:32-48). */
int64_t cueq_gemm_tn_items(int64_t rows, int32_t nparts);
int cueq_gemm_tn(int32_t in_dtype, int64_t M, int64_t N, int64_t rows, const void* A, int64_t lda, int64_t stride_a,
                 const void* B, int64_t ldb, int64_t stride_b, int32_t nparts, float* partials, double alpha, void* stream);

/* out[b][c][r] = in[b][r][c] (layout changes "bijd<->dbij" of _layer_norm_transpose.py:162-227 and operand
 * re-orientation for the incoming direction and the backward contractions).  rows, cols below 2^31, batch below 65536,
 * and at most one of rows / cols beyond 4 194 240 (2 097 120 for 4-byte or odd-sized inputs): the longer one goes to grid.x. */
int cueq_transpose(int32_t dtype, int64_t batch, int64_t rows, int64_t cols, const void* in, void* out, void* stream);

/* Per-segment (u, v) -> (v, u) transposition of every row, one pass: out[r][o] = in[r][src_index[o]] with the row
 * permutation src_index (device, int32, length total) built once by the caller from the segment list.  Stands for the
 * native segmented_transpose op behind cuequivariance_torch/primitives/transpose.py:83-183 (mul_ir <-> ir_mul).
 * element_size 2, 4 or 8 bytes; in and out must not alias. */
int cueq_segmented_transpose(int32_t element_size, int64_t rows, int64_t total, const int32_t* src_index, const void* in, void* out,
                             void* stream);

/* Row LayerNorm with biased variance, rstd = 1/sqrt(var + eps) (_layer_norm_transpose.py:196-209); gamma / beta may
 * be NULL; mean and rstd (float32, one per row) are kept for the backward.  D <= 1024. */
int cueq_layer_norm_fwd(int32_t dtype, int64_t rows, int64_t D, const void* x, const void* gamma, const void* beta,
                        double eps, void* y, float* mean, float* rstd, void* stream);
int64_t cueq_layer_norm_bwd_workspace(int64_t rows, int64_t D);
/* dx from dy, the forward input x and the saved statistics; dgamma / dbeta (float32[D], may be NULL) are summed
 * over rows without atomics through the workspace. */
int cueq_layer_norm_bwd(int32_t dtype, int64_t rows, int64_t D, const void* dy, const void* x, const float* mean,
                        const float* rstd, const void* gamma, void* dx, float* dgamma, float* dbeta, void* workspace,
                        int64_t workspace_bytes, void* stream);

/* LayerNorm over d of a tensor stored d-major, x_t (D x M), into row-major y (M x D), and its backward from
 * dy (M x D) to dx_t (D x M): the LayerNorm with a layout change after the triangular contraction
 * (_layer_norm_transpose.py:162-227) without a transposed copy.  mean, rstd: M floats.  D at most 256; D and M
 * multiples of 16 bytes of elements and 16-byte aligned pointers, else CUEQ_ERR_UNSUPPORTED (use cueq_transpose and the
 * row versions).  The workspace (cueq_layer_norm_t_bwd_workspace bytes) is needed when dgamma or dbeta is asked for. */
int cueq_layer_norm_t_fwd(int32_t dtype, int64_t M, int64_t D, const void* x_t, const void* gamma, const void* beta, double eps,
                          void* y, float* mean, float* rstd, void* stream);
int64_t cueq_layer_norm_t_bwd_workspace(int32_t dtype, int64_t M, int64_t D);
int cueq_layer_norm_t_bwd(int32_t dtype, int64_t M, int64_t D, const void* dy, const void* x_t, const float* mean, const float* rstd,
                          const void* gamma, void* dx_t, float* dgamma, float* dbeta, void* workspace, int64_t workspace_bytes,
                          void* stream);

/* out = sigmoid(u + bias_u) * (v + bias_v) * mask on a rows x cols array (u, v float32 accumulators of the two
 * projections); biases (may be NULL) are indexed by row (bias_axis 0) or column (1), the mask (may be NULL)
 * likewise (_sigmoid_gated_dual_gemm.py:135-150).  cueq_gate_bwd returns the gradients of u and v
 * (_sigmoid_gated_dual_gemm.py:153-218). */
int cueq_gate_fwd(int32_t dtype, int64_t rows, int64_t cols, const float* u, const float* v, const void* bias_u,
                  const void* bias_v, int32_t bias_axis, const void* mask, int32_t mask_axis, void* out, void* stream);
int cueq_gate_bwd(int32_t dtype, int64_t rows, int64_t cols, const void* dout, const float* u, const float* v,
                  const void* bias_u, const void* bias_v, int32_t bias_axis, const void* mask, int32_t mask_axis,
                  void* du, void* dv, void* stream);

/* Deterministic reductions of a rows x cols array into float32: over columns (one value per row) and over rows
 * (one value per column; workspace of cueq_sum_rows_workspace bytes).  Used for bias and affine gradients. */
int cueq_sum_cols(int32_t dtype, int64_t rows, int64_t cols, const void* in, float* out, void* stream);
int64_t cueq_sum_rows_workspace(int64_t rows, int64_t cols);
int cueq_sum_rows(int32_t dtype, int64_t rows, int64_t cols, const void* in, float* out, void* workspace,
                  int64_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CUEQ_AMD_H */
