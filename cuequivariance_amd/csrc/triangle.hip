// Kernels of the triangle multiplicative update (AlphaFold-style pair update):
//   LayerNorm over the hidden dimension, sigmoid-gated dual projection, the triangular contraction
//   t[d,b,i,j] = sum_k a[d,b,i,k] b[d,b,j,k], LayerNorm across d with a layout change, output gate.
// The stages are separate launches composed by the host (cuequivariance_amd/cuet/triangle.py):
//   cueq_gemm_nt        batched C = alpha * A * B^T (+ C), both operands contraction-contiguous, MFMA
//   cueq_transpose      batched 2-D transpose through LDS
//   cueq_layer_norm_*   row LayerNorm forward / backward (one wavefront per row)
//   cueq_gate_*         out = sigmoid(u + bu) * (v + bv) * mask and its backward
//   cueq_sum_rows/cols  reductions for the bias / affine gradients
// Math is fp32 throughout; tensors are fp32 or bf16.
//
// Algorithm reference: cuequivariance_jax/cuequivariance_jax/triangle/_triangle_multiplicative_update.py:371-417,
// _layer_norm_transpose.py:162-227, _sigmoid_gated_dual_gemm.py:111-218 (the torch entry point
// cuequivariance_torch/primitives/triangle.py:138-262 forwards to a closed kernel).

#include <algorithm>

#include "common.h"
#include "cw_common.h"
#include "u1d_spec.h"

namespace cueq {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

__device__ __forceinline__ float tri_load(const float* p, int64_t i) { return p[i]; }
__device__ __forceinline__ float tri_load(const uint16_t* p, int64_t i) { return bf16_bits_to_float(p[i]); }
__device__ __forceinline__ float tri_load(const f16bits* p, int64_t i) { return mm_widen<f16bits>(p[i].bits); }
__device__ __forceinline__ uint16_t raw16(uint16_t v) { return v; }  // the bits of a 2-byte element
__device__ __forceinline__ uint16_t raw16(f16bits v) { return v.bits; }
__device__ __forceinline__ void tri_store(float* p, int64_t i, float v) { p[i] = v; }
__device__ __forceinline__ void tri_store(uint16_t* p, int64_t i, float v) { p[i] = float_to_bf16_bits(v); }
__device__ __forceinline__ void tri_store(f16bits* p, int64_t i, float v) { p[i].bits = mm_round<f16bits>(v); }

// ------------------------------------------------------------------------------------------------
// C[b] (M x N) = alpha * A[b] (M x K, row stride lda) * B[b]^T (N x K, row stride ldb)  (+ C[b])
// 128 x 128 block tile, 4 wavefronts of 64 x 64, 64 bytes of k per row and step, double-buffered LDS.
// Lane half h of a wavefront supplies the same k subset to both MFMA operands, so the k order
// inside a step is free and every operand read is one or two ds_read_b128.
// ------------------------------------------------------------------------------------------------
constexpr int kTile = 128;
constexpr int kRowBytes = 80;  // 64 bytes of data + 16 bytes of padding

// Workgroups are handed to the 8 XCDs round-robin in launch order and every XCD has its own L2.  This maps the
// launch-order index to a tile index so that each XCD works through one contiguous range of tiles (column tile
// fastest, then row tile, then batch): tiles that read the same operand rows then share an L2.
__device__ __forceinline__ void xcd_tile(int& bx, int& by, int& bz) {
  const uint64_t gx = gridDim.x, gy = gridDim.y;
  const uint64_t total = gx * gy * gridDim.z;
  const uint64_t L = blockIdx.x + gx * (blockIdx.y + gy * blockIdx.z);
  const uint64_t q = total >> 3, r = total & 7, x = L & 7;
  const uint64_t P = x * q + (x < r ? x : r) + (L >> 3);
  bx = static_cast<int>(P % gx);
  by = static_cast<int>((P / gx) % gy);
  bz = static_cast<int>(P / (gx * gy));
}

// ------------------------------------------------------------------------------------------------
// Results leave the MFMA register layout (a lane holds one column and 16 rows of a 32 x 32 tile) through LDS, so
// that global memory sees 16-byte vectors on contiguous row segments: 2-byte stores straight from that layout reach
// only a fraction of the write bandwidth.  put: one 32 x 32 accumulator into a staging tile whose rows are
// `row_stride` bytes apart; flush: a wavefront moves 32 rows x NCOLS staged elements to C (optionally adding what is
// there).  A staging tile is private to one wavefront, whose LDS operations execute in program order.
// ------------------------------------------------------------------------------------------------
typedef float floatx2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
// Two floats rounded to nearest even and packed (one conversion instruction), and the halves of such a word as floats;
// F selects the 2-byte format: uint16_t = bfloat16, f16bits = half.
template <typename F>
__device__ __forceinline__ uint32_t pack16(float lo, float hi) { return mm_pack<F>(lo, hi); }
template <typename F>
__device__ __forceinline__ float lo16(uint32_t w) {
  if constexpr (is_half_bits<F>::value) return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(w & 0xffffu)));
  else return __uint_as_float(w << 16);
}
template <typename F>
__device__ __forceinline__ float hi16(uint32_t w) {
  if constexpr (is_half_bits<F>::value) return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(w >> 16)));
  else return __uint_as_float(w & 0xffff0000u);
}

// The value again, as far as the compiler can tell a new one: the two floats of a packed pair are then unpacked where they
// are used instead of being kept, one register each, from the first pass over the data to the last.
__device__ __forceinline__ uint32_t again(uint32_t w) {
  asm volatile("" : "+v"(w));
  return w;
}
// The arithmetic of the LayerNorm statistics over groups of eight elements, spelled out operation by operation (no
// contraction left to the compiler) because two kernels share it and must give the same bits: the row kernel
// ln_fwd_rows8 and the LayerNorm inside dual_gate_res_kernel.
__device__ __forceinline__ float ln_sum8(const float* v) {
  float s = v[0];
#pragma unroll
  for (int e = 1; e < 8; ++e) s = __fadd_rn(s, v[e]);
  return s;
}
__device__ __forceinline__ float ln_center_sq8(float* v, float mu) {  // v -= mu, returns the sum of squares
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = __fsub_rn(v[e], mu);
  float ss = __fmul_rn(v[0], v[0]);
#pragma unroll
  for (int e = 1; e < 8; ++e) ss = fmaf(v[e], v[e], ss);
  return ss;
}
__device__ __forceinline__ float ln_rstd(float sumsq, float inv_d, float eps) { return 1.0f / sqrtf(fmaf(sumsq, inv_d, eps)); }
__device__ __forceinline__ float ln_affine(float centered, float rs, float gm, float bt) {
  return __fadd_rn(__fmul_rn(__fmul_rn(centered, rs), gm), bt);
}

template <typename TO>
__device__ __forceinline__ void stage_put(char* tile, int row_stride, int col, int h, const floatx16& acc, float alpha) {
  using F = TO;
#pragma unroll
  for (int v = 0; v < 16; v += 2) {
    char* p = tile + (8 * (v >> 2) + 4 * h + (v & 3)) * row_stride + col * static_cast<int>(sizeof(TO));
    if constexpr (sizeof(TO) == 2) {
      const uint32_t w = pack16<F>(alpha * acc[v], alpha * acc[v + 1]);
      *reinterpret_cast<uint16_t*>(p) = static_cast<uint16_t>(w & 0xffffu);
      *reinterpret_cast<uint16_t*>(p + row_stride) = static_cast<uint16_t>(w >> 16);
    } else {
      *reinterpret_cast<float*>(p) = alpha * acc[v];
      *reinterpret_cast<float*>(p + row_stride) = alpha * acc[v + 1];
    }
  }
}

template <typename TO>
__device__ __forceinline__ uint4 add_vec(uint4 a, uint4 b) {
  using F = TO;
  if constexpr (sizeof(TO) == 2) {
    const uint32_t x[4] = {a.x, a.y, a.z, a.w}, y[4] = {b.x, b.y, b.z, b.w};
    uint32_t r[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      r[e] = pack16<F>(lo16<F>(x[e]) + lo16<F>(y[e]),
                       hi16<F>(x[e]) + hi16<F>(y[e]));
    return make_uint4(r[0], r[1], r[2], r[3]);
  } else {
    return make_uint4(__float_as_uint(__uint_as_float(a.x) + __uint_as_float(b.x)), __float_as_uint(__uint_as_float(a.y) + __uint_as_float(b.y)),
                      __float_as_uint(__uint_as_float(a.z) + __uint_as_float(b.z)), __float_as_uint(__uint_as_float(a.w) + __uint_as_float(b.w)));
  }
}

// nthreads threads (index t) move `rows` staged rows of NCOLS elements to C (row stride ldc elements)
template <typename TO, int NCOLS>
__device__ __forceinline__ void stage_flush(const char* tile, int row_stride, int rows, TO* __restrict__ C, int64_t ldc, int t, int nthreads,
                                            bool accumulate) {
  constexpr int EPV = 16 / sizeof(TO), VPR = NCOLS / EPV;
  for (int idx = t; idx < rows * VPR; idx += nthreads) {
    const int r = idx / VPR, cv = idx % VPR;
    uint4 val = *reinterpret_cast<const uint4*>(tile + r * row_stride + cv * 16);
    uint4* g = reinterpret_cast<uint4*>(C + static_cast<int64_t>(r) * ldc + cv * EPV);
    if (accumulate) val = add_vec<TO>(val, *g);
    *g = val;
  }
}

// TA / TB: the operand is given contraction-major (K x M resp. K x N, row stride lda / ldb) instead of the default
// contraction-contiguous M x K / N x K.  Such a tile is staged as it lies in memory (rows of k) and the MFMA operand
// is assembled on the way out of LDS: 2-byte types with the transposing read ds_read_b64_tr_b16 (within 16 lanes,
// lane 4g+p receives element p of the four 8-byte rows addressed by lanes g, 4+g, 8+g, 12+g), 4-byte types with
// plain reads along the row.  The row strides (320 / 640 bytes) spread the rows of one read over all banks.
typedef short shortx4_t __attribute__((ext_vector_type(4)));
// bytes between the k rows of a contraction-major tile of EXT columns: the row plus 64 (2-byte) / 128 (4-byte) bytes
template <typename TI, int EXT>
constexpr int trans_stride() { return EXT * static_cast<int>(sizeof(TI)) + (sizeof(TI) == 2 ? 64 : 128); }
// LDS bytes of one operand tile of EXT rows (either layout); KB = bytes of k per row and step (64 or 128), rows of a
// contraction-contiguous tile are KB + 16 bytes apart (conflict-free 16-byte reads by 16 consecutive rows for both)
template <typename TI, int EXT, int KB = 64>
constexpr int gemm_tile_bytes() {
  constexpr int a = EXT * (KB + 16), b = (KB / static_cast<int>(sizeof(TI))) * trans_stride<TI, EXT>();
  return a > b ? a : b;
}

template <typename TI, bool TR, int EXT, int KB = 64>
__device__ __forceinline__ void gemm_stage_offsets(int e, int& row, int& part) {
  constexpr int VPRN = EXT * sizeof(TI) / 16;  // vectors per k row of a contraction-major tile
  if constexpr (TR) { row = e / VPRN; part = e % VPRN; }
  else { row = e / (KB / 16); part = e % (KB / 16); }
}

// fragment of subtile rows [base, base + 32) for MFMA slice q of the step (KB / 32 slices): 16 bytes of k per lane
template <typename TI, bool TR, int EXT, int KB = 64>
__device__ __forceinline__ uint4 gemm_fragment(const char* tile, int base, int q, int lane) {
  constexpr int kTransStride16 = trans_stride<uint16_t, EXT>(), kTransStride32 = trans_stride<float, EXT>();
  constexpr int HK = KB / 2 / static_cast<int>(sizeof(TI));  // k rows of a contraction-major tile per half wavefront
  const int c = lane & 31, h = lane >> 5;
  if constexpr (!TR) {
    return *reinterpret_cast<const uint4*>(tile + (base + c) * (KB + 16) + h * (KB / 2) + q * 16);
  } else if constexpr (sizeof(TI) == 2) {
    const int s = lane & 15, g16 = (lane >> 4) & 1;
    const char* p = tile + (HK * h + 8 * q + (s >> 2)) * kTransStride16 + (base + 16 * g16 + 4 * (s & 3)) * 2;  // k as in the other layout
    typedef shortx4_t __attribute__((address_space(3))) * lptr;
    const shortx4_t r0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(p));
    const shortx4_t r1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(p + 4 * kTransStride16));
    const uint2 a = __builtin_bit_cast(uint2, r0), b = __builtin_bit_cast(uint2, r1);
    return make_uint4(a.x, a.y, b.x, b.y);
  } else {
    const char* p = tile + (HK * h + 4 * q) * kTransStride32 + (base + c) * 4;
    return make_uint4(*reinterpret_cast<const uint32_t*>(p), *reinterpret_cast<const uint32_t*>(p + kTransStride32),
                      *reinterpret_cast<const uint32_t*>(p + 2 * kTransStride32), *reinterpret_cast<const uint32_t*>(p + 3 * kTransStride32));
  }
}

// WM x WN wavefronts of 64 x 64 per block: 2 x 2 (a 128 x 128 tile) by default; 4 x 4 (256 x 256, 16 wavefronts) halves
// the operand traffic between L2 and the CUs for products whose both extents are large.
// KB: bytes of k per row and step; 128 makes every request of a contraction-contiguous operand a whole 128-byte line (with
// 64 a line is fetched in two halves one step apart, and a 256 x 256 step turns over the whole L1 in between).
template <typename TI, typename TO, bool TA, bool TB, int WM = 2, int WN = 2, int KB = 64>
__global__ void __launch_bounds__(64 * WM * WN) gemm_kernel(const TI* __restrict__ A, int64_t lda, int64_t sA,
                                                   const TI* __restrict__ B, int64_t ldb, int64_t sB,
                                                   TO* __restrict__ C, int64_t ldc, int64_t sC, int Mfull, int N, int Kfull,
                                                   float alpha, int accumulate, int vec_out, int64_t k_total, int nparts, int64_t pA,
                                                   int64_t pB, int64_t pC, const int64_t* __restrict__ goff, int ngroups, int gmode,
                                                   int64_t gsB, int64_t gsC) {
  using F = TI;
  constexpr int EPV = 16 / sizeof(TI);  // elements per 16-byte vector
  constexpr int BK = KB / sizeof(TI);   // k extent of one step
  constexpr int RB = KB + 16;           // bytes between the rows of a contraction-contiguous tile
  constexpr int NQ = KB / 32;           // 16-byte slices of k per half wavefront and step
  constexpr int TMR = 64 * WM, TNC = 64 * WN, NTH = 64 * WM * WN;  // tile rows, tile columns, threads
  constexpr int TSA = trans_stride<TI, TMR>(), TSB = trans_stride<TI, TNC>();
  constexpr int ABYTES = gemm_tile_bytes<TI, TMR, KB>(), BBYTES = gemm_tile_bytes<TI, TNC, KB>();
  constexpr int NVA = TMR * (KB / 16) / NTH, NVB = TNC * (KB / 16) / NTH;  // 16-byte vectors per thread and step
  __shared__ __align__(16) char smem[2][ABYTES + BBYTES];
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, c = lane & 31, h = lane >> 5;
  const int wm = wave / WN, wn = wave % WN;
  int bx, by, bz;
  xcd_tile(bx, by, bz);
  int m0 = by * TMR, M = Mfull;
  const int n0 = bx * TNC;
  // batch item = (chunk, part): strides s* between chunks, p* between parts (nparts == 1: a plain batch)
  const int chunk = bz / nparts, part = bz - chunk * nparts;
  if (gmode == 3) {  // the parts are unrelated blocks: element offsets of A, B, C per part from a table
    A += static_cast<int64_t>(chunk) * sA + goff[3 * part];
    B += static_cast<int64_t>(chunk) * sB + goff[3 * part + 1];
    C += static_cast<int64_t>(chunk) * sC + goff[3 * part + 2];
  } else {
    A += static_cast<int64_t>(chunk) * sA + static_cast<int64_t>(part) * pA;
    B += static_cast<int64_t>(chunk) * sB + static_cast<int64_t>(part) * pB;
    C += static_cast<int64_t>(chunk) * sC + static_cast<int64_t>(part) * pC;
  }
  // k_total > 0: the chunks are consecutive k ranges of one long contraction; the last ones may be short or empty
  int K = k_total > 0 ? static_cast<int>(max<int64_t>(0, min<int64_t>(Kfull, k_total - static_cast<int64_t>(chunk) * Kfull))) : Kfull;
  if (gmode == 1) {
    // rows grouped: rows [goff[g], goff[g+1]) of A and C use the B of group g; the row-tile index walks the groups'
    // tiles in order (a tile never straddles two groups; the grid has one spare tile per group)
    int t = by, g = 0;
    for (; g < ngroups; ++g) {
      const int64_t lo = goff[g], n = goff[g + 1] - lo;
      const int nt = static_cast<int>((n + TMR - 1) / TMR);
      if (t < nt) {
        m0 = static_cast<int>(lo) + t * TMR;
        break;
      }
      t -= nt;
    }
    if (g == ngroups) return;  // the whole block leaves before any barrier
    M = static_cast<int>(goff[g + 1]);
    B += static_cast<int64_t>(g) * gsB;
  } else if (gmode == 2) {
    // contraction grouped: chunk g contracts rows [goff[g], goff[g+1]) of the contraction-major operands into its own C
    const int64_t k0 = goff[chunk];
    K = static_cast<int>(goff[chunk + 1] - k0);
    A += k0 * lda;
    B += k0 * ldb;
    C += static_cast<int64_t>(chunk) * gsC;
  }

  // every thread stages NVA 16-byte vectors of A and NVB of B per step
  uint4 stA[NVA], stB[NVB];
  int arow[NVA], apart[NVA], brow[NVB], bpart[NVB];
#pragma unroll
  for (int q = 0; q < NVA; ++q) gemm_stage_offsets<TI, TA, TMR, KB>(tid + q * NTH, arow[q], apart[q]);
#pragma unroll
  for (int q = 0; q < NVB; ++q) gemm_stage_offsets<TI, TB, TNC, KB>(tid + q * NTH, brow[q], bpart[q]);
  auto load_one = [&](const TI* __restrict__ P, int64_t ld, bool tr, int row, int part, int x0, int X, int ks) -> uint4 {
    if (tr) {  // row = k within the step, part = vector along the tile's columns (extent X is a multiple of EPV)
      const int k = ks * BK + row, x = x0 + part * EPV;
      const bool ok = k < K && x < X;
      const uint4 v = *reinterpret_cast<const uint4*>(P + static_cast<int64_t>(ok ? k : 0) * ld + (ok ? x : 0));
      return ok ? v : make_uint4(0, 0, 0, 0);
    }
    const int k = ks * BK + part * EPV;
    const bool ok = k < K;
    const uint4 v = *reinterpret_cast<const uint4*>(P + static_cast<int64_t>(min(x0 + row, X - 1)) * ld + (ok ? k : 0));
    return ok ? v : make_uint4(0, 0, 0, 0);
  };
  auto load_step = [&](int ks) {
#pragma unroll
    for (int q = 0; q < NVA; ++q) stA[q] = load_one(A, lda, TA, arow[q], apart[q], m0, M, ks);
#pragma unroll
    for (int q = 0; q < NVB; ++q) stB[q] = load_one(B, ldb, TB, brow[q], bpart[q], n0, N, ks);
  };
  auto store_step = [&](int buf) {
#pragma unroll
    for (int q = 0; q < NVA; ++q) *reinterpret_cast<uint4*>(&smem[buf][arow[q] * (TA ? TSA : RB) + apart[q] * 16]) = stA[q];
#pragma unroll
    for (int q = 0; q < NVB; ++q)
      *reinterpret_cast<uint4*>(&smem[buf][ABYTES + brow[q] * (TB ? TSB : RB) + bpart[q] * 16]) = stB[q];
  };

  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = floatx16{0};

  const int nsteps = (K + BK - 1) / BK;
  if (nsteps > 0) load_step(0);
  int buf = 0;
  for (int ks = 0; ks < nsteps; ++ks) {
    store_step(buf);
    __syncthreads();
    if (ks + 1 < nsteps) load_step(ks + 1);
    uint4 fa[2][NQ], fb[2][NQ];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        fa[t][q] = gemm_fragment<TI, TA, TMR, KB>(&smem[buf][0], wm * 64 + t * 32, q, lane);
        fb[t][q] = gemm_fragment<TI, TB, TNC, KB>(&smem[buf][ABYTES], wn * 64 + t * 32, q, lane);
      }
    // consecutive MFMAs go to different accumulators: a dependent one would wait for its predecessor to drain
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      if constexpr (sizeof(TI) == 2) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j] = mm_32x32x16<F>(fa[i][q], fb[j][q], acc[i][j]);
      } else {
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
          for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(reinterpret_cast<const float*>(&fa[i][q])[s],
                                                               reinterpret_cast<const float*>(&fb[j][q])[s], acc[i][j], 0, 0, 0);
      }
    }
    buf ^= 1;
  }

  // 2-byte results, whole wavefront tile inside C, 16-byte aligned rows: through LDS, 32 rows at a time (4-byte
  // results already leave as 128-byte row segments and gain nothing from the detour)
  if constexpr (sizeof(TO) == 2) {
    __syncthreads();  // every wavefront is done with the operand tiles, which become staging space
    // (parts addressed through a table: every part checks the alignment of its own result block)
    const bool vec_rows = gmode == 3 ? (reinterpret_cast<uintptr_t>(C) % 16 == 0 && (ldc * sizeof(TO)) % 16 == 0) : vec_out != 0;
    if (vec_rows && m0 + wm * 64 + 64 <= M && n0 + wn * 64 + 64 <= N) {
      constexpr int RS = 64 * sizeof(TO) + 16;
      static_assert(WM * WN * 32 * RS <= 2 * (ABYTES + BBYTES), "staging tiles must fit the operand buffers");
      char* tile = &smem[0][0] + wave * (32 * RS);
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        stage_put<TO>(tile, RS, c, h, acc[i][0], alpha);
        stage_put<TO>(tile, RS, 32 + c, h, acc[i][1], alpha);
        __builtin_amdgcn_wave_barrier();
        stage_flush<TO, 64>(tile, RS, 32, C + static_cast<int64_t>(m0 + wm * 64 + i * 32) * ldc + n0 + wn * 64, ldc, lane, 64, accumulate != 0);
        __builtin_amdgcn_wave_barrier();
      }
      return;
    }
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = n0 + wn * 64 + j * 32 + c;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * 64 + i * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
        if (row < M && col < N) {
          const int64_t o = static_cast<int64_t>(row) * ldc + col;
          float val = alpha * acc[i][j][v];
          if (accumulate) val += tri_load(C, o);
          tri_store(C, o, val);
        }
      }
    }
}

// ------------------------------------------------------------------------------------------------
// Partial products of C (M x N) = sum_z A[z, :M]^T B[z, :N] over a long row range: item (chunk, part) of
// grid.z covers rows [chunk * rows_per_chunk, ...) of the column blocks A + part * stride_a, B + part * stride_b
// and writes alpha * partial to P[item] (float32, M x N).  The caller sums the items in order (no atomics).
// Rows are staged through LDS as float32 (bf16 inputs are widened on the way), MFMA 32x32x2 f32.
// ------------------------------------------------------------------------------------------------
constexpr int kTnRows = 16;  // rows (contraction) per step

__device__ __forceinline__ void tn_load8(const float* p, float* r) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  r[0] = a.x; r[1] = a.y; r[2] = a.z; r[3] = a.w; r[4] = b.x; r[5] = b.y; r[6] = b.z; r[7] = b.w;
}
template <typename F>
__device__ __forceinline__ void tn_load8(const F* p, float* r) {
  const uint4 a = *reinterpret_cast<const uint4*>(p);
  const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    r[2 * e] = lo16<F>(w[e]);
    r[2 * e + 1] = hi16<F>(w[e]);
  }
}

template <typename TI, bool VEC>
__global__ void __launch_bounds__(256) gemm_tn_kernel(const TI* __restrict__ A, int64_t lda, int64_t sA, const TI* __restrict__ B,
                                                      int64_t ldb, int64_t sB, float* __restrict__ P, int M, int N, int64_t rows,
                                                      int64_t rows_per_chunk, int nparts, float alpha) {
  using F = TI;
  __shared__ __align__(16) float sa[kTnRows][kTile + 4];
  __shared__ __align__(16) float sb[kTnRows][kTile + 4];
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, c = lane & 31, h = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * kTile, n0 = blockIdx.x * kTile;
  const int64_t item = blockIdx.z;
  const int64_t chunk = item / nparts;
  const int part = static_cast<int>(item - chunk * nparts);
  A += part * sA;
  B += part * sB;
  P += (part * (static_cast<int64_t>(gridDim.z) / nparts) + chunk) * static_cast<int64_t>(M) * N;  // part-major
  const int64_t z_begin = chunk * rows_per_chunk;
  const int64_t z_end = min(z_begin + rows_per_chunk, rows);

  // staging: 16 rows x 128 columns per operand; a thread owns (row, 8 consecutive columns)
  const int srow = tid >> 4, scol = (tid & 15) * 8;
  float ra[8], rb[8];
  auto load_step = [&](int64_t z) {
    const int64_t zr = z + srow;
    if constexpr (VEC) {  // M, N multiples of 8 and 16-byte aligned rows: whole vectors are in or out
      if (zr < z_end && m0 + scol < M) tn_load8(A + zr * lda + m0 + scol, ra);
      else {
#pragma unroll
        for (int e = 0; e < 8; ++e) ra[e] = 0.f;
      }
      if (zr < z_end && n0 + scol < N) tn_load8(B + zr * ldb + n0 + scol, rb);
      else {
#pragma unroll
        for (int e = 0; e < 8; ++e) rb[e] = 0.f;
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const bool ok = zr < z_end;
        ra[e] = (ok && m0 + scol + e < M) ? tri_load(A, zr * lda + m0 + scol + e) : 0.f;
        rb[e] = (ok && n0 + scol + e < N) ? tri_load(B, zr * ldb + n0 + scol + e) : 0.f;
      }
    }
  };
  auto store_step = [&]() {
#pragma unroll
    for (int e = 0; e < 8; e += 4) {
      *reinterpret_cast<float4*>(&sa[srow][scol + e]) = make_float4(ra[e], ra[e + 1], ra[e + 2], ra[e + 3]);
      *reinterpret_cast<float4*>(&sb[srow][scol + e]) = make_float4(rb[e], rb[e + 1], rb[e + 2], rb[e + 3]);
    }
  };

  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = floatx16{0};

  if (z_begin < z_end) load_step(z_begin);
  for (int64_t z = z_begin; z < z_end; z += kTnRows) {
    __syncthreads();  // the previous step's reads are done
    store_step();
    __syncthreads();
    if (z + kTnRows < z_end) load_step(z + kTnRows);
#pragma unroll
    for (int s = 0; s < kTnRows / 2; ++s) {
      const int zr = h * (kTnRows / 2) + s;  // lane half h covers its own half of the rows
      const float a0 = sa[zr][wm * 64 + c], a1 = sa[zr][wm * 64 + 32 + c];
      const float b0 = sb[zr][wn * 64 + c], b1 = sb[zr][wn * 64 + 32 + c];
      acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
      acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
    }
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = n0 + wn * 64 + j * 32 + c;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * 64 + i * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
        if (row < M && col < N) P[static_cast<int64_t>(row) * N + col] = alpha * acc[i][j][v];
      }
    }
}

// ------------------------------------------------------------------------------------------------
// Two products of the same shape and the sigmoid gate in one kernel:
//   u = A1 * B1^T,  v = A2 * B2^T   (A* M x K, B* N x K, contraction contiguous, fp32 accumulate)
//   BWD == false:  C = sigmoid(u + b1) * (v + b2) * mask
//   BWD == true :  dU = dC * mask * (v + b2) * s * (1 - s),  dV = dC * mask * s,   s = sigmoid(u + b1)
// so the two accumulators never travel through memory (the backward recomputes them).  Biases and mask are
// indexed by row (axis 0) or column (axis 1) of C.  Same 128 x 128 tiling as gemm_nt_kernel; SHARE_B: B2 == B1.
// ------------------------------------------------------------------------------------------------
template <typename TI, bool BWD, bool SHARE_B>
__global__ void __launch_bounds__(512, 4) dual_gate_kernel(const TI* __restrict__ A1, const TI* __restrict__ A2, int64_t lda,
                                                           const TI* __restrict__ B1, const TI* __restrict__ B2, int64_t ldb,
                                                           const TI* __restrict__ bias1, const TI* __restrict__ bias2, int bias_axis,
                                                           const TI* __restrict__ mask, int mask_axis, const TI* __restrict__ dC,
                                                           TI* __restrict__ out1, TI* __restrict__ out2, int64_t ldc, int M, int N, int K,
                                                           int vec_out) {
  using F = TI;
  // 8 wavefronts of 64 x 32 (both products): half the accumulators per wavefront of the plain GEMM tiling, so two
  // blocks fit a CU and one block's epilogue overlaps the other's loads.
  constexpr int EPV = 16 / sizeof(TI);
  constexpr int BK = 64 / sizeof(TI);
  constexpr int NT = SHARE_B ? 3 : 4;  // staged tiles per step: A1, A2, B1 (, B2)
  __shared__ __align__(16) char smem[2][NT][kTile * kRowBytes];
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, c = lane & 31, h = lane >> 5;
  const int wm = wave >> 2, wn = wave & 3;
  int bx, by, bz;
  xcd_tile(bx, by, bz);
  const int m0 = by * kTile, n0 = bx * kTile;

  uint4 st[NT];
  const int ldrow = tid >> 2, ldpart = tid & 3;
  const int64_t offa = static_cast<int64_t>(min(m0 + ldrow, M - 1)) * lda + ldpart * EPV;
  const int64_t offb = static_cast<int64_t>(min(n0 + ldrow, N - 1)) * ldb + ldpart * EPV;
  auto load_step = [&](int ks) {
    const int k = ks * BK;
    if (k + ldpart * EPV < K) {
      st[0] = *reinterpret_cast<const uint4*>(A1 + offa + k);
      st[1] = *reinterpret_cast<const uint4*>(A2 + offa + k);
      st[2] = *reinterpret_cast<const uint4*>(B1 + offb + k);
      if constexpr (!SHARE_B) st[3] = *reinterpret_cast<const uint4*>(B2 + offb + k);
    } else {
#pragma unroll
      for (int t = 0; t < NT; ++t) st[t] = make_uint4(0, 0, 0, 0);
    }
  };
  auto store_step = [&](int buf) {
#pragma unroll
    for (int t = 0; t < NT; ++t) *reinterpret_cast<uint4*>(&smem[buf][t][ldrow * kRowBytes + ldpart * 16]) = st[t];
  };

  // the accumulators start from the biases (by row or by column of the result)
  const int col = n0 + wn * 32 + c;
  const int colc = min(col, N - 1);
  floatx16 acc[2][2];  // [product][i]
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const TI* bias = p == 0 ? bias1 : bias2;
    const float cb = (bias && bias_axis == 1) ? tri_load(bias, colc) : 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = min(m0 + wm * 64 + i * 32 + 8 * (v >> 2) + 4 * h + (v & 3), M - 1);
        acc[p][i][v] = (bias && bias_axis == 0) ? tri_load(bias, row) : cb;
      }
  }

  const int nsteps = (K + BK - 1) / BK;
  load_step(0);
  int buf = 0;
  for (int ks = 0; ks < nsteps; ++ks) {
    store_step(buf);
    __syncthreads();
    if (ks + 1 < nsteps) load_step(ks + 1);
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const char* sa = &smem[buf][p][(wm * 64 + c) * kRowBytes + h * 32];
      const char* sb = &smem[buf][(SHARE_B || p == 0) ? 2 : 3][(wn * 32 + c) * kRowBytes + h * 32];
      uint4 fa[2][2], fb[2];
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        fa[0][q] = *reinterpret_cast<const uint4*>(sa + q * 16);
        fa[1][q] = *reinterpret_cast<const uint4*>(sa + 32 * kRowBytes + q * 16);
        fb[q] = *reinterpret_cast<const uint4*>(sb + q * 16);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        if constexpr (sizeof(TI) == 2) {
#pragma unroll
          for (int q = 0; q < 2; ++q)
            acc[p][i] = mm_32x32x16<F>(fa[i][q], fb[q], acc[p][i]);
        } else {
#pragma unroll
          for (int q = 0; q < 2; ++q) {
            const float* pa = reinterpret_cast<const float*>(&fa[i][q]);
            const float* pb = reinterpret_cast<const float*>(&fb[q]);
#pragma unroll
            for (int s2 = 0; s2 < 4; ++s2) acc[p][i] = __builtin_amdgcn_mfma_f32_32x32x2f32(pa[s2], pb[s2], acc[p][i], 0, 0, 0);
          }
        }
      }
    }
    buf ^= 1;
  }

  const float cmk = (mask && mask_axis == 1) ? tri_load(mask, colc) : 1.f;
  const bool rowmk = mask && mask_axis == 0;

  if constexpr (!BWD) {
    // whole block tile inside the output and 16-byte aligned rows: 64 rows at a time through LDS
    if (vec_out && m0 + kTile <= M && n0 + kTile <= N) {
      constexpr int RS = kTile * sizeof(TI) + 16;
      static_assert(64 * RS <= 2 * NT * kTile * kRowBytes, "staging tile must fit the operand buffers");
      char* tile = &smem[0][0][0];
#pragma unroll
      for (int pass = 0; pass < 2; ++pass) {
        __syncthreads();  // operand reads / the previous flush are done
        if (wm == pass) {
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            floatx16 g;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
              const int row = m0 + wm * 64 + i * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
              g[v] = __builtin_amdgcn_rcpf(1.0f + __expf(-acc[0][i][v])) * acc[1][i][v] * (rowmk ? tri_load(mask, row) : cmk);
            }
            stage_put<TI>(tile + i * 32 * RS, RS, wn * 32 + c, h, g, 1.0f);
          }
        }
        __syncthreads();
        stage_flush<TI, kTile>(tile, RS, 64, out1 + static_cast<int64_t>(m0 + pass * 64) * ldc + n0, ldc, tid, 512, false);
      }
      return;
    }
  }
  if (col >= N) return;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int row = m0 + wm * 64 + i * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
      if (row < M) {
        const int64_t o = static_cast<int64_t>(row) * ldc + col;
        const float vv = acc[1][i][v];
        const float sg = __builtin_amdgcn_rcpf(1.0f + __expf(-acc[0][i][v]));
        const float mk = rowmk ? tri_load(mask, row) : cmk;
        if constexpr (!BWD) {
          tri_store(out1, o, sg * vv * mk);
        } else {
          const float d = tri_load(dC, o) * mk;
          tri_store(out1, o, d * vv * sg * (1.0f - sg));
          tri_store(out2, o, d * sg);
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Backward of the gated dual projection down to the projection inputs, in one kernel:
//   u[c][m] = W1[c,:] . X1[m,:],  v[c][m] = W2[c,:] . X2[m,:]        (recomputed, K = 32 * KT)
//   s = sigmoid(u + b1[c]),  d = dC * mask[m],  du = d (v + b2[c]) s (1 - s),  dv = d s
//   dX1[m,:] (+)= sum_c du[c][m] W1[c,:] (+ sum_c dv[c][m] W2[c,:] unless SPLIT),   SPLIT: dX2[m,:] = sum_c dv[c][m] W2[c,:]
// A wavefront owns 32 columns m for the whole kernel and walks the rows c in chunks of 32.  The 32 x 32 MFMA result
// holds, per lane, one m and 16 values of c - exactly an operand of the next MFMA with m as the row and c as the
// contraction - so du and dv go from the accumulator straight into the second product and never touch memory
// (they are written only when the caller asks for them, for the weight gradients).  X fragments stay in registers;
// weight chunks are double-buffered in LDS, row-major; the second product reads them along the columns (2-byte
// types with the transposing LDS read).
// ------------------------------------------------------------------------------------------------
template <typename TI>
__device__ __forceinline__ void mma_step(floatx16& acc, const uint4& a, const uint4& b) {
  using F = TI;
  if constexpr (sizeof(TI) == 2) {
    acc = mm_32x32x16<F>(a, b, acc);
  } else {
    const float* pa = reinterpret_cast<const float*>(&a);
    const float* pb = reinterpret_cast<const float*>(&b);
#pragma unroll
    for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(pa[e], pb[e], acc, 0, 0, 0);
  }
}

// A wavefront-uniform address, pinned to scalar registers so that loads take the "scalar base + 32-bit lane offset" form
// instead of one 64-bit vector address per access.
__device__ __forceinline__ const char* uniform_ptr(const void* p) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
  const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
  return reinterpret_cast<const char*>((static_cast<uint64_t>(hi) << 32) | lo);
}

template <typename V>
__device__ __forceinline__ V load_global(const char* uniform_base, uint32_t lane_offset) {
  typedef const __attribute__((address_space(1))) V* gptr;
  return *reinterpret_cast<gptr>(reinterpret_cast<uint64_t>(uniform_base) + lane_offset);
}
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
template <>
__device__ __forceinline__ uint4 load_global<uint4>(const char* uniform_base, uint32_t lane_offset) {
  const u32x4_t v = load_global<u32x4_t>(uniform_base, lane_offset);
  return make_uint4(v.x, v.y, v.z, v.w);
}
template <>
__device__ __forceinline__ uint2 load_global<uint2>(const char* uniform_base, uint32_t lane_offset) {
  const u32x2_t v = load_global<u32x2_t>(uniform_base, lane_offset);
  return make_uint2(v.x, v.y);
}


// 4 wavefronts (128 columns m) per block; the 2-byte single-input case fits 2 wavefronts per SIMD (two blocks per
// CU, so one block's waits overlap the other's work), the others need more registers and run 1 per SIMD.
template <typename TI, bool SPLIT>
constexpr int gbi_threads() { return 256; }
template <typename TI, bool SPLIT>
constexpr int gbi_waves_per_simd() { return (sizeof(TI) == 2 && !SPLIT) ? 2 : 1; }

// DC_BY_ROW: dC, dU, dV are C x M (else M x C).  Addresses inside the loop are a uniform 64-bit base plus a 32-bit
// lane offset (the host checks the extents), which keeps them out of the vector registers.
template <typename TI, int KT, bool SPLIT, bool DC_BY_ROW>
__global__ void __launch_bounds__((gbi_threads<TI, SPLIT>()), (gbi_waves_per_simd<TI, SPLIT>()))
    gate_bwd_input_kernel(const TI* __restrict__ W1, const TI* __restrict__ W2, int64_t ldw, const TI* __restrict__ X1,
                          const TI* __restrict__ X2, int64_t ldx,
                          const TI* __restrict__ bias1, const TI* __restrict__ bias2, const TI* __restrict__ mask,
                          const TI* __restrict__ dC, int64_t ldc, TI* __restrict__ dX1, TI* __restrict__ dX2,
                          int64_t lddx, int accumulate, TI* __restrict__ dU, TI* __restrict__ dV, int C, int M) {
  using F = TI;
  constexpr bool BF = sizeof(TI) == 2;
  constexpr int EPV = 16 / sizeof(TI);
  constexpr int K = 32 * KT;
  constexpr int ROWB = K * sizeof(TI);  // bytes of one weight row
  constexpr int WSTR = ROWB + 16;       // LDS row stride of a row-major chunk (32 rows)
  constexpr int NS = ROWB / 64;         // 64-byte contraction steps of the first product
  constexpr int WBYTES = 32 * WSTR;
  constexpr int BIAS = 2 * WBYTES;      // offset of the chunk's biases (2 x 32 float)
  constexpr int BUF = BIAS + 256;
  constexpr int NTH = gbi_threads<TI, SPLIT>(), BM = NTH / 2;  // threads and columns m per block
  constexpr int VPR = ROWB / 16, NWV = 32 * VPR, NW = (NWV + NTH - 1) / NTH;
  __shared__ __align__(16) char smem[2][BUF];

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, c = lane & 31, h = lane >> 5;
  const int mcol = blockIdx.x * BM + wave * 32 + c;  // this lane's m in the first product (column) ...
  const int mld = min(mcol, M - 1);
  const int mrow0 = blockIdx.x * BM + wave * 32;     // ... and the wavefront's first m in the second (rows by v)

  constexpr int ES = sizeof(TI);
  uint4 stw[2][NW];
  uint32_t wofs[NW];
#pragma unroll
  for (int q = 0; q < NW; ++q) {
    const int e = min(tid + q * NTH, NWV - 1);
    wofs[q] = static_cast<uint32_t>(((e / VPR) * ldw + (e % VPR) * EPV) * ES);
  }
  // biases of the chunk: threads 0..31 / 32..63 (of every 64) fetch bias1 / bias2, the first 64 threads store them
  const TI* bsrc = (tid & 32) ? bias2 : bias1;
  const bool has_bias = bsrc != nullptr;
  const char* bptr = reinterpret_cast<const char*>(has_bias ? bsrc : W1);
  const uint32_t bofs = has_bias ? static_cast<uint32_t>((tid & 31) * ES) : 0u;
  TI stb;
  // the next chunk and its biases are fetched at the top of an iteration and stored after the first product
  auto load_rows = [&](int c0) {
    stb = *reinterpret_cast<const TI*>(bptr + (has_bias ? static_cast<int64_t>(c0) * ES : 0) + bofs);  // bptr differs by lane
    const char* w1 = uniform_ptr(reinterpret_cast<const char*>(W1) + static_cast<int64_t>(c0) * ldw * ES);
    const char* w2 = uniform_ptr(reinterpret_cast<const char*>(W2) + static_cast<int64_t>(c0) * ldw * ES);
#pragma unroll
    for (int q = 0; q < NW; ++q) {
      stw[0][q] = load_global<uint4>(w1, wofs[q]);
      stw[1][q] = load_global<uint4>(w2, wofs[q]);
    }
  };
  auto store_rows = [&](int buf) {
    if (tid < 64) {
      float bv = 0.f;
      if (has_bias) {
        if constexpr (BF) bv = mm_widen<F>(raw16(stb));
        else bv = stb;
      }
      *reinterpret_cast<float*>(&smem[buf][BIAS + tid * 4]) = bv;
    }
#pragma unroll
    for (int q = 0; q < NW; ++q) {
      const int e = tid + q * NTH;
      if (NWV % NTH == 0 || e < NWV) {
        const int o = (e / VPR) * WSTR + (e % VPR) * 16;
        *reinterpret_cast<uint4*>(&smem[buf][o]) = stw[0][q];
        *reinterpret_cast<uint4*>(&smem[buf][WBYTES + o]) = stw[1][q];
      }
    }
  };
  // fragments of X for this lane's m: lane half h holds bytes [64 s + 32 h, +32) of the row
  uint4 xf1[NS][2], xf2[SPLIT ? NS : 1][2];
#pragma unroll
  for (int s2 = 0; s2 < NS; ++s2)
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int64_t o = static_cast<int64_t>(mld) * ldx + (s2 * 64 + h * 32 + q * 16) / static_cast<int>(sizeof(TI));
      xf1[s2][q] = *reinterpret_cast<const uint4*>(X1 + o);
      if constexpr (SPLIT) xf2[s2][q] = *reinterpret_cast<const uint4*>(X2 + o);
    }
  const float mk = mask ? tri_load(mask, mld) : 1.0f;

  floatx16 ax1[KT], ax2[SPLIT ? KT : 1];
#pragma unroll
  for (int t = 0; t < KT; ++t) ax1[t] = floatx16{0};
#pragma unroll
  for (int t = 0; t < (SPLIT ? KT : 1); ++t) ax2[t] = floatx16{0};

  // cotangent of a chunk: value v of the lane belongs to row c0 + 8 (v >> 2) + 4 h + (v & 3); fetched one chunk ahead
  // (kept as loaded - one register per value, or packed pairs when read along c - and widened where it is used)
  uint32_t dcr[16], dcn[16];
  const uint32_t dcofs = DC_BY_ROW ? static_cast<uint32_t>((4 * h * ldc + mld) * ES) : static_cast<uint32_t>((mld * ldc + 4 * h) * ES);
  auto load_dc = [&](int c0) {
    if constexpr (DC_BY_ROW) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const char* base = uniform_ptr(reinterpret_cast<const char*>(dC) + static_cast<int64_t>(c0 + 8 * (v >> 2) + (v & 3)) * ldc * ES);
        if constexpr (BF) dcn[v] = load_global<uint16_t>(base, dcofs);
        else dcn[v] = load_global<uint32_t>(base, dcofs);
      }
    } else {
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const char* base = uniform_ptr(reinterpret_cast<const char*>(dC) + static_cast<int64_t>(c0 + 8 * a) * ES);
        if constexpr (BF) {
          const uint2 w = load_global<uint2>(base, dcofs);
          dcn[4 * a] = w.x; dcn[4 * a + 1] = w.y;  // values 4a..4a+3 in two registers
        } else {
          const uint4 w = load_global<uint4>(base, dcofs);
          dcn[4 * a] = w.x; dcn[4 * a + 1] = w.y; dcn[4 * a + 2] = w.z; dcn[4 * a + 3] = w.w;
        }
      }
    }
  };
  auto dc_value = [&](int v) -> float {
    if constexpr (!BF) return __uint_as_float(dcr[v]);
    else {
      if constexpr (DC_BY_ROW) return lo16<F>(dcr[v]);
      const uint32_t w = dcr[4 * (v >> 2) + ((v & 3) >> 1)];
      return (v & 1) ? hi16<F>(w) : lo16<F>(w);
    }
  };

  const int nchunks = C / 32;
  load_rows(0);
  load_dc(0);
  store_rows(0);
  __syncthreads();
  for (int ci = 0; ci < nchunks; ++ci) {
    const int c0 = ci * 32, buf = ci & 1;
    const bool more = ci + 1 < nchunks;
#pragma unroll
    for (int v = 0; v < 16; ++v) dcr[v] = dcn[v];
    if (more) {
      load_rows(c0 + 32);
      load_dc(c0 + 32);  // a whole iteration ahead of its use
    }

    // first product: u, v for 32 rows c x 32 columns m; the accumulators start from the biases of their rows
    floatx16 au, av;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const float4 b1 = *reinterpret_cast<const float4*>(&smem[buf][BIAS + (8 * a + 4 * h) * 4]);
      const float4 b2 = *reinterpret_cast<const float4*>(&smem[buf][BIAS + 128 + (8 * a + 4 * h) * 4]);
      au[4 * a] = b1.x; au[4 * a + 1] = b1.y; au[4 * a + 2] = b1.z; au[4 * a + 3] = b1.w;
      av[4 * a] = b2.x; av[4 * a + 1] = b2.y; av[4 * a + 2] = b2.z; av[4 * a + 3] = b2.w;
    }
    {
      const char* w1 = &smem[buf][c * WSTR + h * 32];
#pragma unroll
      for (int s2 = 0; s2 < NS; ++s2)
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          const uint4 a1 = *reinterpret_cast<const uint4*>(w1 + s2 * 64 + q * 16);
          const uint4 a2 = *reinterpret_cast<const uint4*>(w1 + WBYTES + s2 * 64 + q * 16);
          mma_step<TI>(au, a1, xf1[s2][q]);
          mma_step<TI>(av, a2, SPLIT ? xf2[s2][q] : xf1[s2][q]);
        }
    }

    if (more) store_rows(buf ^ 1);  // the other buffer was last read before the previous barrier

    // gate backward in registers; du, dv are packed (2-byte types) as soon as they exist
    float du[BF ? 4 : 16], dv[BF ? 4 : 16];
    uint32_t pu[BF ? 8 : 1], pv[BF ? 8 : 1];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int v = 4 * a + b;
        const float uu = au[v], vv = av[v];
        const float sg = __builtin_amdgcn_rcpf(1.0f + __expf(-uu));
        const float dvv = dc_value(v) * mk * sg;           // dv = d s
        const float duv = dvv * fmaf(-vv, sg, vv);          // du = d v s (1 - s)
        du[BF ? b : v] = duv;
        dv[BF ? b : v] = dvv;
        if (dU != nullptr && mcol < M) {
          const int row = c0 + 8 * a + 4 * h + b;
          const int64_t o = DC_BY_ROW ? static_cast<int64_t>(row) * ldc + mcol : static_cast<int64_t>(mcol) * ldc + row;
          tri_store(dU, o, duv);
          tri_store(dV, o, dvv);
        }
      }
      if constexpr (BF) {
        pu[2 * a] = pack16<F>(du[0], du[1]); pu[2 * a + 1] = pack16<F>(du[2], du[3]);
        pv[2 * a] = pack16<F>(dv[0], dv[1]); pv[2 * a + 1] = pack16<F>(dv[2], dv[3]);
      }
    }
    // second product: rows m (lanes of the operand), contraction over the 32 rows c of the chunk
    if constexpr (BF) {
      // operand of the second product: for column d = 32 ds + (lane & 31), the 8 rows c that this lane's du / dv
      // values belong to (16 t + 4 h + 0..3 and + 8), gathered from the row-major chunk by two transposing reads
      typedef shortx4_t __attribute__((address_space(3))) * lptr;
      const int s16 = lane & 15, g16 = (lane >> 4) & 1;
      const char* t1 = &smem[buf][(4 * h + (s16 >> 2)) * WSTR + (16 * g16 + 4 * (s16 & 3)) * 2];
#pragma unroll
      for (int ds = 0; ds < KT; ++ds)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const char* p1 = t1 + t * 16 * WSTR + ds * 64;
          const uint2 l1 = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(p1)));
          const uint2 h1 = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(p1 + 8 * WSTR)));
          const uint2 l2 = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(p1 + WBYTES)));
          const uint2 h2 = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(p1 + WBYTES + 8 * WSTR)));
          mma_step<TI>(ax1[ds], make_uint4(pu[4 * t], pu[4 * t + 1], pu[4 * t + 2], pu[4 * t + 3]), make_uint4(l1.x, l1.y, h1.x, h1.y));
          mma_step<TI>(SPLIT ? ax2[ds] : ax1[ds], make_uint4(pv[4 * t], pv[4 * t + 1], pv[4 * t + 2], pv[4 * t + 3]),
                       make_uint4(l2.x, l2.y, h2.x, h2.y));
        }
    } else {
#pragma unroll
      for (int ds = 0; ds < KT; ++ds)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const char* p1 = &smem[buf][(8 * (v >> 2) + 4 * h + (v & 3)) * WSTR + (ds * 32 + c) * 4];
          const float w1 = *reinterpret_cast<const float*>(p1), w2 = *reinterpret_cast<const float*>(p1 + WBYTES);
          ax1[ds] = __builtin_amdgcn_mfma_f32_32x32x2f32(du[v], w1, ax1[ds], 0, 0, 0);
          if constexpr (SPLIT) ax2[ds] = __builtin_amdgcn_mfma_f32_32x32x2f32(dv[v], w2, ax2[ds], 0, 0, 0);
          else ax1[ds] = __builtin_amdgcn_mfma_f32_32x32x2f32(dv[v], w2, ax1[ds], 0, 0, 0);
        }
    }

    __syncthreads();
  }

  // (the loop's last barrier has passed: the weight buffers are free for staging)
  if (mrow0 + 32 <= M) {
    constexpr int RS = ROWB + 16;
    static_assert(4 * 32 * RS <= 2 * BUF, "staging tiles must fit the weight buffers");
    char* tile = &smem[0][0] + wave * (32 * RS);
#pragma unroll
    for (int ds = 0; ds < KT; ++ds) stage_put<TI>(tile, RS, ds * 32 + c, h, ax1[ds], 1.0f);
    __builtin_amdgcn_wave_barrier();
    stage_flush<TI, K>(tile, RS, 32, dX1 + static_cast<int64_t>(mrow0) * lddx, lddx, lane, 64, accumulate != 0);
    if constexpr (SPLIT) {
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int ds = 0; ds < KT; ++ds) stage_put<TI>(tile, RS, ds * 32 + c, h, ax2[ds], 1.0f);
      __builtin_amdgcn_wave_barrier();
      stage_flush<TI, K>(tile, RS, 32, dX2 + static_cast<int64_t>(mrow0) * lddx, lddx, lane, 64, false);
    }
    return;
  }
#pragma unroll
  for (int ds = 0; ds < KT; ++ds) {
    const int col = ds * 32 + c;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int row = mrow0 + 8 * (v >> 2) + 4 * h + (v & 3);
      if (row < M) {
        const int64_t o = static_cast<int64_t>(row) * lddx + col;
        float val = ax1[ds][v];
        if (accumulate) val += tri_load(dX1, o);
        tri_store(dX1, o, val);
        if constexpr (SPLIT) tri_store(dX2, o, ax2[ds][v]);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// The same computation for 2-byte types with the weights resident in LDS: one block per CU loads W1, W2 (C rows)
// and the biases once, then its wavefronts walk 32-column tiles of m independently - no barrier and no weight
// traffic inside the loop, and wavefronts of one SIMD drift into different phases (MFMA / gate math / memory).
// LDS: 2 C (2 K + 16) bytes of weights + 8 C bytes of biases (+ with two inputs a wave-private 8-row staging tile for the results).
//
// LNB (one-input form): X1 holds the rows of a LayerNorm whose input rows, mean and 1 / std are given, and the kernel
// goes on to the gradient with respect to those input rows - the lane has half of the gradient row in registers, so the two
// row sums of the LayerNorm backward are sums over its own values completed by one exchange - and writes that to dX1.
// ------------------------------------------------------------------------------------------------
template <typename F, int KT, bool SPLIT, bool DC_BY_ROW, bool LNB = false>
__global__ void __launch_bounds__((SPLIT ? 256 : 512), (SPLIT ? 1 : 2))
    gate_bwd_input_res_kernel(const F* __restrict__ W1, const F* __restrict__ W2, int64_t ldw, const F* __restrict__ X1,
                              const F* __restrict__ X2, int64_t ldx, const F* __restrict__ bias1,
                              const F* __restrict__ bias2, const F* __restrict__ mask, const F* __restrict__ dC,
                              int64_t ldc, F* __restrict__ dX1, F* __restrict__ dX2, int64_t lddx, int accumulate,
                              F* __restrict__ dU, F* __restrict__ dV, int C, int M, const F* __restrict__ ln_x = nullptr,
                              int64_t ldlx = 0, const float* __restrict__ ln_mean = nullptr, const float* __restrict__ ln_rstd = nullptr,
                              const F* __restrict__ ln_gamma = nullptr) {
  static_assert(!(LNB && SPLIT), "the LayerNorm backward goes with the one-input form");
  using TI = F;
  constexpr int ES = 2, EPV = 8;
  constexpr int K = 32 * KT, ROWB = K * ES, NS = ROWB / 64, VPR = ROWB / 16;
  // weight rows in LDS: 256-byte rows keep their 16-byte units XOR-swizzled by a rotation of the row's low four bits
  // (16 consecutive rows put one unit on 16 different bank groups for the row-operand reads; 4 consecutive rows put
  // one 64-byte span on 4 different ones for the transposing reads); shorter rows are padded by 16 bytes instead
  constexpr bool SWZ = KT == 4;
  constexpr int WSTR = SWZ ? ROWB : ROWB + 16, SSTR = ROWB + 16;
  auto swz = [](int row) -> int { return SWZ ? (((row & 3) << 2) | ((row >> 2) & 3)) : 0; };
  constexpr int NTH = SPLIT ? 256 : 512, NWAVES = NTH / 64;
  extern __shared__ __align__(16) char gbi_dsm[];
  char* sw1 = gbi_dsm;
  char* sw2 = gbi_dsm + C * WSTR;
  float* sb = reinterpret_cast<float*>(gbi_dsm + 2 * C * WSTR);  // bias1[C], bias2[C]
  const int tid = threadIdx.x;
  // (the wavefront's number as a scalar: tile indices and row bases derived from it stay in scalar registers)
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, c = lane & 31, h = lane >> 5;
  char* stage = reinterpret_cast<char*>(sb + 2 * C) + wave * (8 * SSTR);  // (two inputs only)
  float* sg = sb + 2 * C;                                                   // (LNB only) gamma[K]

  for (int e = tid; e < C * VPR; e += NTH) {
    const int r = e / VPR, part = e % VPR;
    const int po = (part ^ swz(r)) << 4;
    *reinterpret_cast<uint4*>(sw1 + r * WSTR + po) = *reinterpret_cast<const uint4*>(W1 + static_cast<int64_t>(r) * ldw + part * EPV);
    *reinterpret_cast<uint4*>(sw2 + r * WSTR + po) = *reinterpret_cast<const uint4*>(W2 + static_cast<int64_t>(r) * ldw + part * EPV);
  }
  for (int i = tid; i < C; i += NTH) {
    sb[i] = bias1 ? tri_load(bias1, i) : 0.f;
    sb[C + i] = bias2 ? tri_load(bias2, i) : 0.f;
  }
  if constexpr (LNB) {
    for (int i = tid; i < K; i += NTH) sg[i] = ln_gamma ? tri_load(ln_gamma, i) : 1.f;
  }
  __syncthreads();

  const int nchunks = C / 32;
  const int64_t ntiles = (static_cast<int64_t>(M) + 31) / 32;
  // v_perm_b32 selectors (bytes 0-3 = own register, 4-7 = the neighbour's): even lane (own.lo, other.lo), odd lane (other.hi, own.hi)
  const uint32_t pair_sel = (lane & 1) ? 0x03020706u : 0x05040100u;
  const int64_t tstep = static_cast<int64_t>(gridDim.x) * NWAVES;
  auto tile_row = [&](int64_t t) -> int { return static_cast<int>(min(t * 32 + c, static_cast<int64_t>(M) - 1)); };

  // cotangent values of a chunk, packed: register 2 a + j holds rows 8 a + 4 h + 2 j, + 1 of this lane's column.
  // dC by rows (C x M): a lane pair loads 4-byte column pairs - the even lane of row 2 j, the odd lane of row
  // 2 j + 1 - and swaps halves on use; dC by columns (M x C): the four rows are 8 adjacent bytes.
  // The loads run a chunk ahead of their use, across tile boundaries: (ptile, pci) is the next chunk to request.
  uint32_t dcr[8], dcn[8];
  auto dc_lane_offset = [&](int mld) -> uint32_t {
    return DC_BY_ROW ? static_cast<uint32_t>(((4 * h + (lane & 1)) * ldc + (mld & ~1)) * ES) : static_cast<uint32_t>((mld * ldc + 4 * h) * ES);
  };
  int64_t ptile = static_cast<int64_t>(blockIdx.x) * NWAVES + wave;
  int pci = 0;
  uint32_t pofs = ptile < ntiles ? dc_lane_offset(tile_row(ptile)) : 0u;
  auto request_dc = [&](uint32_t (&dst)[8]) {
    if (ptile >= ntiles) return;
    const int c0 = pci * 32;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      if constexpr (DC_BY_ROW) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const char* base = uniform_ptr(reinterpret_cast<const char*>(dC) + static_cast<int64_t>(c0 + 8 * a + 2 * j) * ldc * ES);
          dst[2 * a + j] = load_global<uint32_t>(base, pofs);
        }
      } else {
        const char* base = uniform_ptr(reinterpret_cast<const char*>(dC) + static_cast<int64_t>(c0 + 8 * a) * ES);
        const uint2 w = load_global<uint2>(base, pofs);
        dst[2 * a] = w.x; dst[2 * a + 1] = w.y;
      }
    }
    if (++pci == nchunks) {
      pci = 0;
      ptile += tstep;
      if (ptile < ntiles) pofs = dc_lane_offset(tile_row(ptile));
    }
  };
  auto dc_value = [&](int v) -> float {
    const uint32_t w = dcr[v >> 1];
    return (v & 1) ? hi16<F>(w) : lo16<F>(w);
  };
  // the rows of X of a tile, one row per lane, and its mask value (as stored: converted where it is used, so that the
  // request is not followed by a wait).  The registers are free once the last chunk's first product has read them:
  // the rows of the wavefront's next tile are requested then, and arrive while the results of this one leave.
  uint4 xf1[NS][2], xf2[SPLIT ? NS : 1][2];
  uint32_t mraw = 0;
  auto request_x = [&](int mld) {
#pragma unroll
    for (int s2 = 0; s2 < NS; ++s2)
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const int64_t o = static_cast<int64_t>(mld) * ldx + (s2 * 64 + h * 32 + q * 16) / ES;
        xf1[s2][q] = *reinterpret_cast<const uint4*>(X1 + o);
        if constexpr (SPLIT) xf2[s2][q] = *reinterpret_cast<const uint4*>(X2 + o);
      }
    if (mask) mraw = raw16(mask[mld]);
  };
  int64_t tile = ptile;
  if (tile < ntiles) request_x(tile_row(tile));
  request_dc(dcn);

  for (; tile < ntiles; tile += tstep) {
    const int mrow0 = static_cast<int>(tile * 32);
    const int mcol = mrow0 + c;
    const float mk = mask ? lo16<F>(mraw) : 1.0f;
    floatx16 ax1[KT], ax2[SPLIT ? KT : 1];
#pragma unroll
    for (int t = 0; t < KT; ++t) ax1[t] = floatx16{0};
#pragma unroll
    for (int t = 0; t < (SPLIT ? KT : 1); ++t) ax2[t] = floatx16{0};

    for (int ci = 0; ci < nchunks; ++ci) {
      const int c0 = ci * 32;
#pragma unroll
      for (int v = 0; v < 8; ++v) {
        if constexpr (DC_BY_ROW) {
          const uint32_t other = static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(dcn[v]), 0xB1, 0xF, 0xF, true));
          dcr[v] = __builtin_amdgcn_perm(other, dcn[v], pair_sel);
        } else {
          dcr[v] = dcn[v];
        }
      }
      request_dc(dcn);

      floatx16 au, av;
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const float4 b1 = *reinterpret_cast<const float4*>(sb + c0 + 8 * a + 4 * h);
        const float4 b2 = *reinterpret_cast<const float4*>(sb + C + c0 + 8 * a + 4 * h);
        au[4 * a] = b1.x; au[4 * a + 1] = b1.y; au[4 * a + 2] = b1.z; au[4 * a + 3] = b1.w;
        av[4 * a] = b2.x; av[4 * a + 1] = b2.y; av[4 * a + 2] = b2.z; av[4 * a + 3] = b2.w;
      }
      {
        const int wrow = (c0 + c) * WSTR;
#pragma unroll
        for (int s2 = 0; s2 < NS; ++s2)
#pragma unroll
          for (int q = 0; q < 2; ++q) {
            const int wo = wrow + ((((2 * h + q) ^ swz(c)) << 4) ^ (s2 << 6));
            const uint4 a1 = *reinterpret_cast<const uint4*>(sw1 + wo);
            const uint4 a2 = *reinterpret_cast<const uint4*>(sw2 + wo);
            mma_step<TI>(au, a1, xf1[s2][q]);
            mma_step<TI>(av, a2, SPLIT ? xf2[s2][q] : xf1[s2][q]);
          }
      }
      uint32_t pu[8], pv[8];
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        float du[4], dv[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const int v = 4 * a + b;
          const float sg = __builtin_amdgcn_rcpf(1.0f + __expf(-au[v]));
          dv[b] = dc_value(v) * mk * sg;
          du[b] = dv[b] * fmaf(-av[v], sg, av[v]);
        }
        pu[2 * a] = pack16<F>(du[0], du[1]); pu[2 * a + 1] = pack16<F>(du[2], du[3]);
        pv[2 * a] = pack16<F>(dv[0], dv[1]); pv[2 * a + 1] = pack16<F>(dv[2], dv[3]);
        if (dU != nullptr) {
          const int row = c0 + 8 * a + 4 * h;
          if constexpr (!DC_BY_ROW) {
            // the lane's four rows are adjacent elements of its m row: one 8-byte store per array
            if (mcol < M) {
              const int64_t o = static_cast<int64_t>(mcol) * ldc + row;
              *reinterpret_cast<uint2*>(dU + o) = make_uint2(pu[2 * a], pu[2 * a + 1]);
              *reinterpret_cast<uint2*>(dV + o) = make_uint2(pv[2 * a], pv[2 * a + 1]);
            }
          } else {
            // neighbouring lanes swap halves: the even lane stores rows 0 and 2 for columns (m, m + 1), the odd
            // lane rows 1 and 3 for columns (m - 1, m) - 4-byte stores, 128 contiguous bytes per half-wave
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              const uint32_t ou = pu[2 * a + j], ov = pv[2 * a + j];
              const uint32_t ru = static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(ou), 0xB1, 0xF, 0xF, true));
              const uint32_t rv = static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(ov), 0xB1, 0xF, 0xF, true));
              const uint32_t wu = __builtin_amdgcn_perm(ru, ou, pair_sel), wv = __builtin_amdgcn_perm(rv, ov, pair_sel);
              if (mcol < M) {
                const int64_t o = static_cast<int64_t>(row + 2 * j + (lane & 1)) * ldc + (mcol & ~1);
                *reinterpret_cast<uint32_t*>(dU + o) = wu;
                *reinterpret_cast<uint32_t*>(dV + o) = wv;
              }
            }
          }
        }
      }
      {
        typedef shortx4_t __attribute__((address_space(3))) * lptr;
        const int s16 = lane & 15, g16 = (lane >> 4) & 1;
        // rows 4 h + (s16 >> 2) (+ 8, + 16 t): a row 8 further flips bit 1 of the swizzle, 16 further leaves it
        const int trow = 4 * h + (s16 >> 2), tunit = 2 * g16 + ((s16 & 3) >> 1);
        const int off = (c0 + trow) * WSTR + 8 * (s16 & 1);
        const int ulo = (tunit ^ swz(trow)) << 4, uhi = SWZ ? (ulo ^ 32) : ulo;
#pragma unroll
        for (int ds = 0; ds < KT; ++ds)
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            const int o = off + t * 16 * WSTR + (ulo ^ (ds << 6));
            const int o8 = off + (t * 16 + 8) * WSTR + (uhi ^ (ds << 6));
            const uint2 l1 = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(sw1 + o)));
            const uint2 h1 = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(sw1 + o8)));
            const uint2 l2 = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(sw2 + o)));
            const uint2 h2 = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(sw2 + o8)));
            const uint4 w1f = make_uint4(l1.x, l1.y, h1.x, h1.y), w2f = make_uint4(l2.x, l2.y, h2.x, h2.y);
            const uint4 duf = make_uint4(pu[4 * t], pu[4 * t + 1], pu[4 * t + 2], pu[4 * t + 3]);
            const uint4 dvf = make_uint4(pv[4 * t], pv[4 * t + 1], pv[4 * t + 2], pv[4 * t + 3]);
            if constexpr (SPLIT) {  // a lane of the result holds one k and 16 values of m
              mma_step<TI>(ax1[ds], duf, w1f);
              mma_step<TI>(ax2[ds], dvf, w2f);
            } else {  // the weight columns are the rows of the product: a lane holds its own m and 16 values of k
              mma_step<TI>(ax1[ds], w1f, duf);
              mma_step<TI>(ax1[ds], w2f, dvf);
            }
          }
      }
    }

    // the rows of the next tile (past the end: the last tile again, so that the request is unconditional)
    request_x(tile_row(min(tile + tstep, ntiles - 1)));
    if constexpr (SPLIT) {
      // Results of the two-input form (one wavefront per SIMD, nothing to add to): 8 rows (one value group a) at a time
      // through the wave-private staging tile, whole rows out as 16-byte vectors.  (The stores from registers of the
      // other form, 32 bytes per row and instruction, measure 5 % slower here.)
#pragma unroll
      for (int which = 0; which < 2; ++which) {
        F* dst = which == 0 ? dX1 : dX2;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int ds = 0; ds < KT; ++ds) {
            const floatx16& acc = (which == 0) ? ax1[ds] : ax2[ds];
            const uint32_t w01 = pack16<F>(acc[4 * a], acc[4 * a + 1]), w23 = pack16<F>(acc[4 * a + 2], acc[4 * a + 3]);
            char* p = stage + (4 * h) * SSTR + (ds * 32 + c) * 2;
            *reinterpret_cast<uint16_t*>(p) = static_cast<uint16_t>(w01 & 0xffffu);
            *reinterpret_cast<uint16_t*>(p + SSTR) = static_cast<uint16_t>(w01 >> 16);
            *reinterpret_cast<uint16_t*>(p + 2 * SSTR) = static_cast<uint16_t>(w23 & 0xffffu);
            *reinterpret_cast<uint16_t*>(p + 3 * SSTR) = static_cast<uint16_t>(w23 >> 16);
          }
          __builtin_amdgcn_wave_barrier();
          const int r0 = mrow0 + 8 * a;
          const int rows = min(8, M - r0);
          if (rows > 0) stage_flush<TI, K>(stage, SSTR, rows, dst + static_cast<int64_t>(r0) * lddx, lddx, lane, 64, false);
        }
      }
    } else {
      // Results of the one-input form.  A lane holds row m = mrow0 + c and, per 32 columns, k = 8 (v >> 2) + 4 h + (v & 3):
      // the lane halves swap register pairs (v_permlane32_swap: lanes 32-63 of the first register with lanes 0-31 of the
      // second), after which the lower half has k 0-7 and the upper half k 8-15 of every 16 columns - 16 contiguous bytes
      // per lane, 32 per row and instruction, straight from the registers.  What the results are added to is requested
      // first, in the same shape, all of it at once.  All vectors are formed before the first of them is stored.
      const int mrow = mrow0 + c;
      const int64_t orow = static_cast<int64_t>(min(mrow, M - 1)) * lddx + (h * 16) / ES;
      uint4 old[KT][2];
      if (accumulate) {
#pragma unroll
        for (int ds = 0; ds < KT; ++ds)
#pragma unroll
          for (int j = 0; j < 2; ++j) old[ds][j] = *reinterpret_cast<const uint4*>(dX1 + orow + (ds * 64 + j * 32) / ES);
      }
      uint4 val[KT][2];
      if constexpr (LNB) {
        // dx = rstd (g - mean(g) - xn mean(g xn)) with g = dy gamma, xn = (x - mean) rstd, over the K elements of the row.
        // The float accumulators are swapped into row order (k = 16 j + 8 h + e per 32 columns), what is added to them
        // and the LayerNorm's input rows arrive in the same order.
        uint4 xr[KT][2];
        const int64_t xrow = static_cast<int64_t>(min(mrow, M - 1)) * ldlx + (h * 16) / ES;
#pragma unroll
        for (int ds = 0; ds < KT; ++ds)
#pragma unroll
          for (int j = 0; j < 2; ++j) xr[ds][j] = *reinterpret_cast<const uint4*>(ln_x + xrow + (ds * 64 + j * 32) / ES);
        const float mu = ln_mean[min(mrow, M - 1)], rs = ln_rstd[min(mrow, M - 1)];
        float s1 = 0, s2 = 0;
#pragma unroll
        for (int ds = 0; ds < KT; ++ds) {
          floatx16& acc = ax1[ds];
#pragma unroll
          for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[8 * j + i]), __float_as_uint(acc[8 * j + 4 + i]), false, false);
              acc[8 * j + i] = __uint_as_float(sw[0]);
              acc[8 * j + 4 + i] = __uint_as_float(sw[1]);
            }
            const int k0 = ds * 32 + j * 16 + h * 8;
            const float4 g0 = *reinterpret_cast<const float4*>(sg + k0), g1 = *reinterpret_cast<const float4*>(sg + k0 + 4);
            const float gm[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
            const uint32_t ow[4] = {old[ds][j].x, old[ds][j].y, old[ds][j].z, old[ds][j].w};
            const uint32_t xw[4] = {xr[ds][j].x, xr[ds][j].y, xr[ds][j].z, xr[ds][j].w};
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              float d = acc[8 * j + e];
              if (accumulate) d += (e & 1) ? hi16<F>(ow[e >> 1]) : lo16<F>(ow[e >> 1]);
              const float g = d * gm[e];
              const float xn = (((e & 1) ? hi16<F>(xw[e >> 1]) : lo16<F>(xw[e >> 1])) - mu) * rs;
              s1 += g;
              s2 = fmaf(g, xn, s2);
              acc[8 * j + e] = g;
            }
          }
        }
        s1 = (s1 + __shfl_xor(s1, 32, 64)) * (1.0f / K);
        s2 = (s2 + __shfl_xor(s2, 32, 64)) * (1.0f / K);
#pragma unroll
        for (int ds = 0; ds < KT; ++ds) {
          const floatx16& acc = ax1[ds];
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const uint32_t xw[4] = {again(xr[ds][j].x), again(xr[ds][j].y), again(xr[ds][j].z), again(xr[ds][j].w)};
            uint32_t o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float x0 = (lo16<F>(xw[e]) - mu) * rs, x1 = (hi16<F>(xw[e]) - mu) * rs;
              o[e] = pack16<F>(rs * (acc[8 * j + 2 * e] - s1 - x0 * s2), rs * (acc[8 * j + 2 * e + 1] - s1 - x1 * s2));
            }
            val[ds][j] = make_uint4(o[0], o[1], o[2], o[3]);
          }
        }
      } else {
#pragma unroll
      for (int ds = 0; ds < KT; ++ds) {
        const floatx16& acc = ax1[ds];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const uint32_t p0 = pack16<F>(acc[8 * j], acc[8 * j + 1]), p1 = pack16<F>(acc[8 * j + 2], acc[8 * j + 3]);
          const uint32_t p2 = pack16<F>(acc[8 * j + 4], acc[8 * j + 5]), p3 = pack16<F>(acc[8 * j + 6], acc[8 * j + 7]);
          const auto s0 = __builtin_amdgcn_permlane32_swap(p0, p2, false, false);
          const auto s1 = __builtin_amdgcn_permlane32_swap(p1, p3, false, false);
          val[ds][j] = make_uint4(s0[0], s1[0], s0[1], s1[1]);
          if (accumulate) val[ds][j] = add_vec<TI>(val[ds][j], old[ds][j]);
        }
      }
      }
      __builtin_amdgcn_sched_barrier(0);
      if (mrow < M) {
#pragma unroll
        for (int ds = 0; ds < KT; ++ds)
#pragma unroll
          for (int j = 0; j < 2; ++j) *reinterpret_cast<uint4*>(dX1 + orow + (ds * 64 + j * 32) / ES) = val[ds][j];
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

// ------------------------------------------------------------------------------------------------
// sigmoid(W1 X^T + b1) * (W2 X^T + b2) * mask for 2-byte types with W1, W2 (C rows) and the biases resident in LDS, the
// forward twin of the kernel above: rows c of the result are weight rows, columns m are rows of X; one persistent
// block per CU, every wavefront walks tiles of 64 columns m on its own (two 32-column MFMA tiles sharing each weight
// fragment).  Results leave as 4-byte column pairs: neighbouring lanes swap halves (even lane: row 2 j for columns
// m, m + 1; odd lane: row 2 j + 1 for m - 1, m), so N and ldc must be even.
//
// ROWS: two inputs (W1 meets X, W2 meets X2) and the result by rows, M x C - the output stage of the triangle update.
//
// LN: X holds the rows before their LayerNorm.  A lane has half of its row in registers (the other half is in the lane
// 32 further), so the statistics are sums over the lane's own values completed by one exchange; the rows are
// normalised in the registers, rounded to the 2-byte type - the operand of the products, exactly what a separate
// LayerNorm launch would have written - and stored with their mean and 1 / std for the later stages.
// ------------------------------------------------------------------------------------------------
template <typename F, int KT, bool LN, bool ROWS>
__global__ void __launch_bounds__(512, 2)
    dual_gate_res_kernel(const F* __restrict__ W1, const F* __restrict__ W2, int64_t ldw, const F* __restrict__ X,
                         const F* __restrict__ X2, int64_t ldx, const F* __restrict__ bias1, const F* __restrict__ bias2, const F* __restrict__ mask,
                         F* __restrict__ out, int64_t ldc, int C, int M, const F* __restrict__ gamma,
                         const F* __restrict__ beta, float eps, F* __restrict__ xhat, int64_t ldxh, float* __restrict__ mean,
                         float* __restrict__ rstd) {
  using TI = F;
  constexpr int ES = 2, EPV = 8;
  constexpr int K = 32 * KT, ROWB = K * ES, NS = ROWB / 64, VPR = ROWB / 16;
  constexpr bool SWZ = KT == 4;  // (same layout of the weight rows as gate_bwd_input_res_kernel)
  constexpr int WSTR = SWZ ? ROWB : ROWB + 16;
  constexpr int NTH = 512, NWAVES = NTH / 64;
  constexpr int NT = ROWS ? 1 : 2;  // 32-row MFMA tiles per step of a wavefront (two inputs: one, their rows take the registers)
  static_assert(!(LN && ROWS), "the LayerNorm variant has one input");
  auto swz = [](int row) -> int { return SWZ ? (((row & 3) << 2) | ((row >> 2) & 3)) : 0; };
  extern __shared__ __align__(16) char dgr_dsm[];
  char* sw1 = dgr_dsm;
  char* sw2 = dgr_dsm + C * WSTR;
  float* sb = reinterpret_cast<float*>(dgr_dsm + 2 * C * WSTR);  // bias1[C], bias2[C]
  float* sg = sb + 2 * C;                                           // LN: gamma[K], beta[K]
  const int tid = threadIdx.x;
  // (the wavefront's number as a scalar: tile indices and row bases derived from it stay in scalar registers)
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, c = lane & 31, h = lane >> 5;

  for (int e = tid; e < C * VPR; e += NTH) {
    const int r = e / VPR, part = e % VPR;
    const int po = (part ^ swz(r)) << 4;
    *reinterpret_cast<uint4*>(sw1 + r * WSTR + po) = *reinterpret_cast<const uint4*>(W1 + static_cast<int64_t>(r) * ldw + part * EPV);
    *reinterpret_cast<uint4*>(sw2 + r * WSTR + po) = *reinterpret_cast<const uint4*>(W2 + static_cast<int64_t>(r) * ldw + part * EPV);
  }
  for (int i = tid; i < C; i += NTH) {
    sb[i] = bias1 ? tri_load(bias1, i) : 0.f;
    sb[C + i] = bias2 ? tri_load(bias2, i) : 0.f;
  }
  if constexpr (LN) {
    for (int i = tid; i < K; i += NTH) {
      sg[i] = gamma ? tri_load(gamma, i) : 1.f;
      sg[K + i] = beta ? tri_load(beta, i) : 0.f;
    }
  }
  __syncthreads();

  const int nchunks = C / 32;
  const int64_t ntiles = (static_cast<int64_t>(M) + 32 * NT - 1) / (32 * NT);
  const int64_t tstep = static_cast<int64_t>(gridDim.x) * NWAVES;
  const uint32_t pair_sel = (lane & 1) ? 0x03020706u : 0x05040100u;
  // the rows of a tile, one row per lane (and the lane 32 further), with their mask values as stored; those of the
  // wavefront's next tile are requested while the current one is worked on
  uint4 xn[NT][NS][2], xn2[1][NS][2];
  uint32_t mraw[NT] = {};
  auto request_x = [&](int64_t tl) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int mld = static_cast<int>(min(tl * (32 * NT) + 32 * t + c, static_cast<int64_t>(M) - 1));
#pragma unroll
      for (int s2 = 0; s2 < NS; ++s2)
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          const int64_t o = static_cast<int64_t>(mld) * ldx + (s2 * 64 + h * 32 + q * 16) / ES;
          xn[t][s2][q] = *reinterpret_cast<const uint4*>(X + o);
          if constexpr (ROWS) xn2[t][s2][q] = *reinterpret_cast<const uint4*>(X2 + o);
        }
      if (mask) mraw[t] = raw16(mask[mld]);
    }
  };
  // (tiles dealt out wavefront-major: the tiles worked on at one time lie next to each other in memory and are spread over
  // all CUs - 3 us less per launch than with the eight tiles of a block next to each other)
  const int64_t tile0 = static_cast<int64_t>(wave) * gridDim.x + blockIdx.x;
  if (tile0 < ntiles) request_x(tile0);
  for (int64_t tile = tile0; tile < ntiles; tile += tstep) {
    uint4 xf[NT][NS][2], xf2[1][NS][2];
    float mk[NT];
    int mcol[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      mcol[t] = static_cast<int>(tile * (32 * NT)) + 32 * t + c;
#pragma unroll
      for (int s2 = 0; s2 < NS; ++s2)
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          xf[t][s2][q] = xn[t][s2][q];
          if constexpr (ROWS) xf2[t][s2][q] = xn2[t][s2][q];
        }
      mk[t] = mask ? lo16<F>(mraw[t]) : 1.0f;
    }
    request_x(min(tile + tstep, ntiles - 1));  // (past the end: the last tile again, so that the request is unconditional)
    if constexpr (LN) {
      // The sums are formed in the order of the row kernel ln_fwd_rows8 - groups of eight elements summed in sequence,
      // then pairs, fours, eights of groups - so that both give the same bits: a group pair lives in one lane, the
      // neighbouring pair in the lane 32 further.
      auto tree = [&](const float (&gs)[NS][2]) -> float {
        float quad[NS];
#pragma unroll
        for (int s2 = 0; s2 < NS; ++s2) {
          const float pair = gs[s2][0] + gs[s2][1];
          quad[s2] = pair + __shfl_xor(pair, 32, 64);
        }
        if constexpr (NS == 1) return quad[0];
        else if constexpr (NS == 2) return quad[0] + quad[1];
        else if constexpr (NS == 3) return (quad[0] + quad[1]) + quad[2];
        else return (quad[0] + quad[1]) + (quad[2] + quad[3]);
      };
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        float gs[NS][2];
#pragma unroll
        for (int s2 = 0; s2 < NS; ++s2)
#pragma unroll
          for (int q = 0; q < 2; ++q) {
            const uint32_t w[4] = {xf[t][s2][q].x, xf[t][s2][q].y, xf[t][s2][q].z, xf[t][s2][q].w};
            const float v[8] = {lo16<F>(w[0]), hi16<F>(w[0]), lo16<F>(w[1]), hi16<F>(w[1]), lo16<F>(w[2]), hi16<F>(w[2]), lo16<F>(w[3]), hi16<F>(w[3])};
            gs[s2][q] = ln_sum8(v);
          }
        const float mu = __fmul_rn(tree(gs), 1.0f / K);
#pragma unroll
        for (int s2 = 0; s2 < NS; ++s2)
#pragma unroll
          for (int q = 0; q < 2; ++q) {
            const uint32_t w[4] = {again(xf[t][s2][q].x), again(xf[t][s2][q].y), again(xf[t][s2][q].z), again(xf[t][s2][q].w)};
            float v[8] = {lo16<F>(w[0]), hi16<F>(w[0]), lo16<F>(w[1]), hi16<F>(w[1]), lo16<F>(w[2]), hi16<F>(w[2]), lo16<F>(w[3]), hi16<F>(w[3])};
            gs[s2][q] = ln_center_sq8(v, mu);
          }
        const float rs = ln_rstd(tree(gs), 1.0f / K, eps);
        const int mld = min(mcol[t], M - 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s2 = 0; s2 < NS; ++s2)
#pragma unroll
          for (int q = 0; q < 2; ++q) {
            const int k0 = s2 * 32 + h * 16 + q * 8;
            const float4 g0 = *reinterpret_cast<const float4*>(sg + k0), g1 = *reinterpret_cast<const float4*>(sg + k0 + 4);
            const float4 b0 = *reinterpret_cast<const float4*>(sg + K + k0), b1 = *reinterpret_cast<const float4*>(sg + K + k0 + 4);
            const float gm[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w}, bt[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
            const uint32_t w[4] = {again(xf[t][s2][q].x), again(xf[t][s2][q].y), again(xf[t][s2][q].z), again(xf[t][s2][q].w)};
            uint32_t o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e)
              o[e] = pack16<F>(ln_affine(__fsub_rn(lo16<F>(w[e]), mu), rs, gm[2 * e], bt[2 * e]),
                               ln_affine(__fsub_rn(hi16<F>(w[e]), mu), rs, gm[2 * e + 1], bt[2 * e + 1]));
            xf[t][s2][q] = make_uint4(o[0], o[1], o[2], o[3]);
            if (mcol[t] < M) *reinterpret_cast<uint4*>(xhat + static_cast<int64_t>(mld) * ldxh + (s2 * 64 + h * 32 + q * 16) / ES) = xf[t][s2][q];
            __builtin_amdgcn_sched_barrier(0);  // one piece at a time: its gamma / beta values die here
          }
        if (h == 0 && mcol[t] < M) {
          mean[mld] = mu;
          rstd[mld] = rs;
        }
      }
    }
    for (int ci = 0; ci < nchunks; ++ci) {
      const int c0 = ci * 32;
      floatx16 au[NT], av[NT];
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const float4 b1 = *reinterpret_cast<const float4*>(sb + c0 + 8 * a + 4 * h);
        const float4 b2 = *reinterpret_cast<const float4*>(sb + C + c0 + 8 * a + 4 * h);
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          au[t][4 * a] = b1.x; au[t][4 * a + 1] = b1.y; au[t][4 * a + 2] = b1.z; au[t][4 * a + 3] = b1.w;
          av[t][4 * a] = b2.x; av[t][4 * a + 1] = b2.y; av[t][4 * a + 2] = b2.z; av[t][4 * a + 3] = b2.w;
        }
      }
      const int wrow = (c0 + c) * WSTR;
#pragma unroll
      for (int s2 = 0; s2 < NS; ++s2)
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          const int wo = wrow + ((((2 * h + q) ^ swz(c)) << 4) ^ (s2 << 6));
          const uint4 a1 = *reinterpret_cast<const uint4*>(sw1 + wo);
          const uint4 a2 = *reinterpret_cast<const uint4*>(sw2 + wo);
#pragma unroll
          for (int t = 0; t < NT; ++t) {
            mma_step<TI>(au[t], a1, xf[t][s2][q]);
            mma_step<TI>(av[t], a2, ROWS ? xf2[t][s2][q] : xf[t][s2][q]);
          }
        }
      if constexpr (ROWS) {
        // result by rows (M x C): the lane holds its own row m and, of this chunk, c = 8 (v >> 2) + 4 h + (v & 3); the lane
        // halves swap register pairs (v_permlane32_swap), after which each stores 16 contiguous bytes of its row
        uint32_t pk[8];
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          float g[4];
#pragma unroll
          for (int b = 0; b < 4; ++b) {
            const int v = 4 * a + b;
            g[b] = __builtin_amdgcn_rcpf(1.0f + __expf(-au[0][v])) * av[0][v] * mk[0];
          }
          pk[2 * a] = pack16<F>(g[0], g[1]);
          pk[2 * a + 1] = pack16<F>(g[2], g[3]);
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const auto s0 = __builtin_amdgcn_permlane32_swap(pk[4 * j], pk[4 * j + 2], false, false);
          const auto s1 = __builtin_amdgcn_permlane32_swap(pk[4 * j + 1], pk[4 * j + 3], false, false);
          if (mcol[0] < M)
            *reinterpret_cast<uint4*>(out + static_cast<int64_t>(mcol[0]) * ldc + c0 + 16 * j + 8 * h) = make_uint4(s0[0], s1[0], s0[1], s1[1]);
        }
      } else {
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          float g[4];
#pragma unroll
          for (int b = 0; b < 4; ++b) {
            const int v = 4 * a + b;
            g[b] = __builtin_amdgcn_rcpf(1.0f + __expf(-au[t][v])) * av[t][v] * mk[t];
          }
          const uint32_t own[2] = {pack16<F>(g[0], g[1]), pack16<F>(g[2], g[3])};
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const uint32_t other = static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(own[j]), 0xB1, 0xF, 0xF, true));
            const uint32_t word = __builtin_amdgcn_perm(other, own[j], pair_sel);
            if (mcol[t] < M) {
              const int row = c0 + 8 * a + 4 * h + 2 * j + (lane & 1);
              *reinterpret_cast<uint32_t*>(out + static_cast<int64_t>(row) * ldc + (mcol[t] & ~1)) = word;
            }
          }
        }
      }
    }
  }
}

// any shape / alignment / operand order: one thread per output element (rs*: stride between rows of the operand,
// ks*: stride along the contraction)
template <typename TI, typename TO>
__global__ void __launch_bounds__(256) gemm_simple(const TI* __restrict__ A, int64_t rsa, int64_t ksa, int64_t sA, const TI* __restrict__ B,
                                                   int64_t rsb, int64_t ksb, int64_t sB, TO* __restrict__ C, int64_t ldc, int64_t sC,
                                                   int M, int N, int K, float alpha, int accumulate) {
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tid >= static_cast<int64_t>(M) * N) return;
  const int row = static_cast<int>(tid / N), col = static_cast<int>(tid - static_cast<int64_t>(row) * N);
  A += static_cast<int64_t>(blockIdx.z) * sA + static_cast<int64_t>(row) * rsa;
  B += static_cast<int64_t>(blockIdx.z) * sB + static_cast<int64_t>(col) * rsb;
  C += static_cast<int64_t>(blockIdx.z) * sC;
  float acc = 0;
  for (int k = 0; k < K; ++k) acc = fmaf(tri_load(A, k * ksa), tri_load(B, k * ksb), acc);
  const int64_t o = static_cast<int64_t>(row) * ldc + col;
  float val = alpha * acc;
  if (accumulate) val += tri_load(C, o);
  tri_store(C, o, val);
}

// ------------------------------------------------------------------------------------------------
// batched transpose  out[b][c][r] = in[b][r][c]  (32 x 32 tiles through LDS)
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256) transpose_kernel(const T* __restrict__ in, T* __restrict__ out, int R, int Ccols, int rows_on_x) {
  __shared__ T tile[32][33];
  const int64_t base = static_cast<int64_t>(blockIdx.z) * R * Ccols;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
  // (grid.y holds at most 65535 tiles: the host puts the row tiles on grid.x when there are more)
  const int r0 = (rows_on_x ? blockIdx.x : blockIdx.y) * 32, c0 = (rows_on_x ? blockIdx.y : blockIdx.x) * 32;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int r = r0 + ty + q * 8, cc = c0 + tx;
    if (r < R && cc < Ccols) tile[ty + q * 8][tx] = in[base + static_cast<int64_t>(r) * Ccols + cc];
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int cc = c0 + ty + q * 8, r = r0 + tx;
    if (r < R && cc < Ccols) out[base + static_cast<int64_t>(cc) * R + r] = tile[tx][ty + q * 8];
  }
}

// 2-byte elements, even extents: 64 x 64 tiles moved as pairs (4-byte accesses on both sides)
__global__ void __launch_bounds__(256) transpose16_kernel(const uint16_t* __restrict__ in, uint16_t* __restrict__ out, int R, int Ccols, int rows_on_x) {
  __shared__ uint16_t tile[64][66];
  const int64_t base = static_cast<int64_t>(blockIdx.z) * R * Ccols;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 pairs x 8
  const int r0 = (rows_on_x ? blockIdx.x : blockIdx.y) * 64, c0 = (rows_on_x ? blockIdx.y : blockIdx.x) * 64;
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    const int r = r0 + ty + q * 8, cc = c0 + 2 * tx;
    if (r < R && cc < Ccols) {
      const uint32_t v = *reinterpret_cast<const uint32_t*>(in + base + static_cast<int64_t>(r) * Ccols + cc);
      tile[ty + q * 8][2 * tx] = static_cast<uint16_t>(v & 0xffffu);
      tile[ty + q * 8][2 * tx + 1] = static_cast<uint16_t>(v >> 16);
    }
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    const int cc = c0 + ty + q * 8, r = r0 + 2 * tx;
    if (r < R && cc < Ccols) {
      const uint32_t v = static_cast<uint32_t>(tile[2 * tx][ty + q * 8]) | (static_cast<uint32_t>(tile[2 * tx + 1][ty + q * 8]) << 16);
      *reinterpret_cast<uint32_t*>(out + base + static_cast<int64_t>(cc) * R + r) = v;
    }
  }
}

// ------------------------------------------------------------------------------------------------
// LayerNorm over rows of length D (D <= 1024): one wavefront per row, biased variance
// ------------------------------------------------------------------------------------------------
constexpr int kLnMaxPerLane = 16;

template <typename T, int NQ>
__global__ void __launch_bounds__(256) ln_fwd_kernel(const T* __restrict__ x, const T* __restrict__ gamma, const T* __restrict__ beta,
                                                     T* __restrict__ y, float* __restrict__ mean, float* __restrict__ rstd,
                                                     int64_t rows, int D, float eps) {
  const int lane = threadIdx.x & 63;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T* xr = x + row * D;
  float v[NQ];
  float s = 0;
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int e = lane + q * 64;
    v[q] = e < D ? tri_load(xr, e) : 0.f;
    s += v[q];
  }
  const float mu = wave_sum(s) / D;
  float ss = 0;
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int e = lane + q * 64;
    const float d = e < D ? v[q] - mu : 0.f;
    ss += d * d;
  }
  const float rs = 1.0f / sqrtf(wave_sum(ss) / D + eps);
  T* yr = y + row * D;
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int e = lane + q * 64;
    if (e < D) {
      float o = (v[q] - mu) * rs;
      if (gamma) o *= tri_load(gamma, e);
      if (beta) o += tri_load(beta, e);
      tri_store(yr, e, o);
    }
  }
  if (lane == 0) {
    mean[row] = mu;
    rstd[row] = rs;
  }
}

// dx = rstd * (g - mean(g) - xhat * mean(g * xhat)),  g = dy * gamma;   per-block partial sums of
// dgamma = sum dy * xhat and dbeta = sum dy go to part[2][blocks][D].
template <typename T, int NQ>
__global__ void __launch_bounds__(256) ln_bwd_kernel(const T* __restrict__ dy, const T* __restrict__ x, const float* __restrict__ mean,
                                                     const float* __restrict__ rstd, const T* __restrict__ gamma,
                                                     T* __restrict__ dx, float* __restrict__ part, int64_t rows, int D,
                                                     int rows_per_block) {
  extern __shared__ float sred[];  // [4 waves][2][D]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float ag[NQ], ab[NQ];
#pragma unroll
  for (int q = 0; q < NQ; ++q) ag[q] = ab[q] = 0.f;
  const int64_t r_begin = static_cast<int64_t>(blockIdx.x) * rows_per_block;
  const int64_t r_end = min(r_begin + rows_per_block, rows);
  for (int64_t row = r_begin + wave; row < r_end; row += 4) {
    const T* xr = x + row * D;
    const T* gr = dy + row * D;
    const float mu = mean[row], rs = rstd[row];
    float xh[NQ], g[NQ];
    float s1 = 0, s2 = 0;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      const int e = lane + q * 64;
      if (e < D) {
        xh[q] = (tri_load(xr, e) - mu) * rs;
        const float d = tri_load(gr, e);
        ag[q] += d * xh[q];
        ab[q] += d;
        g[q] = gamma ? d * tri_load(gamma, e) : d;
        s1 += g[q];
        s2 += g[q] * xh[q];
      } else {
        xh[q] = g[q] = 0.f;
      }
    }
    s1 = wave_sum(s1) / D;
    s2 = wave_sum(s2) / D;
    T* dr = dx + row * D;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      const int e = lane + q * 64;
      if (e < D) tri_store(dr, e, rs * (g[q] - s1 - xh[q] * s2));
    }
  }
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int e = lane + q * 64;
    if (e < D) {
      sred[(wave * 2 + 0) * D + e] = ag[q];
      sred[(wave * 2 + 1) * D + e] = ab[q];
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < 2 * D; e += 256) {
    const int which = e / D, d = e - which * D;
    float s = 0;
    for (int w = 0; w < 4; ++w) s += sred[(w * 2 + which) * D + d];
    part[(static_cast<int64_t>(which) * gridDim.x + blockIdx.x) * D + d] = s;
  }
}

// ---- rows of D = 8 L elements: L lanes per row, 8 consecutive elements (16 or 32 bytes) per lane, 64 / L rows
//      per wavefront; reductions stay inside the L lanes ------------------------------------------------------------
__device__ __forceinline__ void ln_store8(float* p, const float* r) {
  *reinterpret_cast<float4*>(p) = make_float4(r[0], r[1], r[2], r[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(r[4], r[5], r[6], r[7]);
}
template <typename F>
__device__ __forceinline__ void ln_store8(F* p, const float* r) {
  uint4 o;
  o.x = mm_round<F>(r[0]) | (static_cast<uint32_t>(mm_round<F>(r[1])) << 16);
  o.y = mm_round<F>(r[2]) | (static_cast<uint32_t>(mm_round<F>(r[3])) << 16);
  o.z = mm_round<F>(r[4]) | (static_cast<uint32_t>(mm_round<F>(r[5])) << 16);
  o.w = mm_round<F>(r[6]) | (static_cast<uint32_t>(mm_round<F>(r[7])) << 16);
  *reinterpret_cast<uint4*>(p) = o;
}
template <int L>
__device__ __forceinline__ float group_sum(float v) {  // sum over aligned groups of L lanes, valid in every lane
  if (L >= 2) v += dpp_move<0xB1>(v);
  if (L >= 4) v += dpp_move<0x4E>(v);
  if (L >= 8) v += dpp_move<0x141>(v);
  if (L >= 16) v += dpp_move<0x140>(v);
  if (L >= 32) v += __shfl_xor(v, 16, 64);
  if (L >= 64) v += __shfl_xor(v, 32, 64);
  return v;
}

template <typename T, int L>
__global__ void __launch_bounds__(256) ln_fwd_rows8(const T* __restrict__ x, const T* __restrict__ gamma, const T* __restrict__ beta,
                                                    T* __restrict__ y, float* __restrict__ mean, float* __restrict__ rstd, int64_t rows,
                                                    float eps) {
  using F = T;
  constexpr int D = 8 * L, RPW = 64 / L;
  const int lane = threadIdx.x & 63, sub = lane / L, col = (lane % L) * 8;
  const int64_t row = (static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6)) * RPW + sub;
  const bool ok = row < rows;
  float v[8], gm[8], bt[8];
  if (ok) tn_load8(x + row * D + col, v);
  else {
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = 0.f;
  }
  const float mu = __fmul_rn(group_sum<L>(ln_sum8(v)), 1.0f / D);
  const float rs = ln_rstd(group_sum<L>(ln_center_sq8(v, mu)), 1.0f / D, eps);
#pragma unroll
  for (int e = 0; e < 8; ++e) gm[e] = 1.f, bt[e] = 0.f;
  if (gamma) tn_load8(gamma + col, gm);
  if (beta) tn_load8(beta + col, bt);
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = ln_affine(v[e], rs, gm[e], bt[e]);
  if (ok) {
    ln_store8(y + row * D + col, v);
    if (lane % L == 0) {
      mean[row] = mu;
      rstd[row] = rs;
    }
  }
}

template <typename T, int L>
__global__ void __launch_bounds__(256) ln_bwd_rows8(const T* __restrict__ dy, const T* __restrict__ x, const float* __restrict__ mean,
                                                    const float* __restrict__ rstd, const T* __restrict__ gamma, T* __restrict__ dx,
                                                    float* __restrict__ part, int64_t rows, int rows_per_block) {
  using F = T;
  constexpr int D = 8 * L, RPW = 64 / L;
  extern __shared__ float sred[];  // [4 waves][2][D]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, sub = lane / L, col = (lane % L) * 8;
  float ag[8], ab[8], gm[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) ag[e] = ab[e] = 0.f;
  if (gamma) tn_load8(gamma + col, gm);
  const int64_t r_begin = static_cast<int64_t>(blockIdx.x) * rows_per_block;
  const int64_t r_end = min(r_begin + rows_per_block, rows);
  for (int64_t r0 = r_begin + wave * RPW; r0 < r_end; r0 += 4 * RPW) {
    const int64_t row = r0 + sub;
    const bool ok = row < r_end;
    float xh[8], g[8];
    float mu = 0.f, rs = 0.f;
    if (ok) {
      tn_load8(x + row * D + col, xh);
      tn_load8(dy + row * D + col, g);
      mu = mean[row];
      rs = rstd[row];
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) xh[e] = g[e] = 0.f;
    }
    float s1 = 0, s2 = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      xh[e] = (xh[e] - mu) * rs;
      ag[e] += g[e] * xh[e];
      ab[e] += g[e];
      if (gamma) g[e] *= gm[e];
      s1 += g[e];
      s2 += g[e] * xh[e];
    }
    s1 = group_sum<L>(s1) * (1.0f / D);
    s2 = group_sum<L>(s2) * (1.0f / D);
#pragma unroll
    for (int e = 0; e < 8; ++e) g[e] = rs * (g[e] - s1 - xh[e] * s2);
    if (ok) ln_store8(dx + row * D + col, g);
  }
  // rows of one wavefront -> one lane group, then the four wavefronts through LDS
#pragma unroll
  for (int e = 0; e < 8; ++e) {
#pragma unroll
    for (int off = L; off < 64; off *= 2) {
      ag[e] += __shfl_xor(ag[e], off, 64);
      ab[e] += __shfl_xor(ab[e], off, 64);
    }
  }
  if (lane < L) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      sred[(wave * 2 + 0) * D + col + e] = ag[e];
      sred[(wave * 2 + 1) * D + col + e] = ab[e];
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < 2 * D; e += 256) {
    const int which = e / D, d = e - which * D;
    float s = 0;
    for (int w = 0; w < 4; ++w) s += sred[(w * 2 + which) * D + d];
    part[(static_cast<int64_t>(which) * gridDim.x + blockIdx.x) * D + d] = s;
  }
}

// ------------------------------------------------------------------------------------------------
// LayerNorm over d of a tensor stored d-major, x_t (D x M, row d contiguous in m), with the result row-major
// y (M x D): the "LayerNorm with a layout change" of the triangle update (_layer_norm_transpose.py:162-227) in one
// pass instead of a transpose and a row LayerNorm.  A block takes MT = 128 / sizeof(T) bytes-worth of consecutive m
// (64 two-byte or 32 four-byte elements: 128-byte row segments of x_t) for all d through an LDS tile.
// The backward takes dy (M x D) and x_t and writes dx_t (D x M); blocks walk tiles with a stride so that the
// gamma / beta partial sums stay few.
// ------------------------------------------------------------------------------------------------
constexpr int kLnTMaxD = 256;
template <typename T>
struct LnT {
  static constexpr int MT = 128 / sizeof(T);       // m per tile
  static constexpr int RS = 132;                   // bytes between d rows of the x tile (33 dwords: no bank conflicts along d)
  static constexpr int G = 256 / MT;               // thread groups along d
  static constexpr int EPV = 16 / sizeof(T);
};

template <typename T>
__device__ __forceinline__ float lnt_tile(const char* tile, int d, int m) {
  using F = T;
  if constexpr (sizeof(T) == 2) return mm_widen<F>(*reinterpret_cast<const uint16_t*>(tile + d * LnT<T>::RS + m * 2));
  else return *reinterpret_cast<const float*>(tile + d * LnT<T>::RS + m * 4);
}

// x_t tile [D][MT] -> LDS (vectors beyond M are zero)
template <typename T>
__device__ __forceinline__ void lnt_load_tile(char* tile, const T* __restrict__ xt, int64_t M, int D, int64_t m0, int tid) {
  constexpr int VPRM = 8;  // 16-byte vectors per 128-byte row segment
  for (int idx = tid; idx < D * VPRM; idx += 256) {
    const int d = idx / VPRM, v = idx % VPRM;
    const int64_t m = m0 + v * LnT<T>::EPV;
    uint4 val = make_uint4(0, 0, 0, 0);
    if (m < M) val = *reinterpret_cast<const uint4*>(xt + static_cast<int64_t>(d) * M + m);
    uint32_t* p = reinterpret_cast<uint32_t*>(tile + d * LnT<T>::RS + v * 16);
    p[0] = val.x; p[1] = val.y; p[2] = val.z; p[3] = val.w;
  }
}

template <typename T>
__global__ void __launch_bounds__(256) ln_t_fwd_kernel(const T* __restrict__ xt, const T* __restrict__ gamma, const T* __restrict__ beta,
                                                       T* __restrict__ y, float* __restrict__ mean, float* __restrict__ rstd, int64_t M, int D,
                                                       float eps) {
  using F = T;
  using L = LnT<T>;
  extern __shared__ __align__(16) char lnt_dyn[];  // D * RS bytes: the x tile
  char* tile = lnt_dyn;
  __shared__ float red[L::G][L::MT];
  __shared__ float smean[L::MT], srstd[L::MT];
  __shared__ __align__(16) float sgam[kLnTMaxD], sbet[kLnTMaxD];
  const int tid = threadIdx.x;
  const int64_t m0 = static_cast<int64_t>(blockIdx.x) * L::MT;
  lnt_load_tile<T>(tile, xt, M, D, m0, tid);
  if (tid < D) {
    sgam[tid] = gamma ? tri_load(gamma, tid) : 1.0f;
    sbet[tid] = beta ? tri_load(beta, tid) : 0.0f;
  }
  __syncthreads();
  const int m = tid % L::MT, g = tid / L::MT;
  float s = 0;
  for (int d = g; d < D; d += L::G) s += lnt_tile<T>(tile, d, m);
  red[g][m] = s;
  __syncthreads();
  if (tid < L::MT) {
    float t = 0;
#pragma unroll
    for (int k = 0; k < L::G; ++k) t += red[k][tid];
    smean[tid] = t / D;
  }
  __syncthreads();
  const float mu = smean[m];
  s = 0;
  for (int d = g; d < D; d += L::G) {
    const float c = lnt_tile<T>(tile, d, m) - mu;
    s += c * c;
  }
  red[g][m] = s;
  __syncthreads();
  if (tid < L::MT) {
    float t = 0;
#pragma unroll
    for (int k = 0; k < L::G; ++k) t += red[k][tid];
    const float r = rsqrtf(t / D + eps);
    srstd[tid] = r;
    if (m0 + tid < M) {
      mean[m0 + tid] = smean[tid];
      rstd[m0 + tid] = r;
    }
  }
  __syncthreads();
  // rows of y: 16-byte vectors along d
  const int vpr = D / L::EPV;
  for (int idx = tid; idx < L::MT * vpr; idx += 256) {
    const int r = idx / vpr, v = idx % vpr;
    if (m0 + r >= M) continue;
    const float mu2 = smean[r], rs = srstd[r];
    float o[L::EPV];
#pragma unroll
    for (int e = 0; e < L::EPV; ++e) {
      const int d = v * L::EPV + e;
      o[e] = (lnt_tile<T>(tile, d, r) - mu2) * rs * sgam[d] + sbet[d];
    }
    uint4 out;
    if constexpr (sizeof(T) == 2) out = make_uint4(pack16<F>(o[0], o[1]), pack16<F>(o[2], o[3]), pack16<F>(o[4], o[5]), pack16<F>(o[6], o[7]));
    else out = make_uint4(__float_as_uint(o[0]), __float_as_uint(o[1]), __float_as_uint(o[2]), __float_as_uint(o[3]));
    *reinterpret_cast<uint4*>(y + (m0 + r) * D + v * L::EPV) = out;
  }
}

template <typename T>
__global__ void __launch_bounds__(256) ln_t_bwd_kernel(const T* __restrict__ dy, const T* __restrict__ xt, const float* __restrict__ mean,
                                                       const float* __restrict__ rstd, const T* __restrict__ gamma, T* __restrict__ dxt,
                                                       float* __restrict__ part, int64_t M, int D, int64_t ntiles, int need_affine) {
  using F = T;
  using L = LnT<T>;
  constexpr int PW = 4 / sizeof(T);  // elements per 4-byte store along m
  extern __shared__ __align__(16) char lnt_dyn[];  // the x tile (D * RS bytes, rounded up to 16), then the dy tile (MT * DS)
  char* tile = lnt_dyn;
  char* dtile = lnt_dyn + ((D * L::RS + 15) & ~15);
  __shared__ float red1[L::G][L::MT], red2[L::G][L::MT];
  __shared__ float smean[L::MT], srstd[L::MT], c1[L::MT], c2[L::MT];
  __shared__ float sgam[kLnTMaxD];
  const int tid = threadIdx.x;
  if (tid < D) sgam[tid] = gamma ? tri_load(gamma, tid) : 1.0f;  // visible after the first barrier of the tile loop
  const int DS = D * static_cast<int>(sizeof(T)) + 4;  // bytes between rows of the dy tile
  const int vpr = D / L::EPV;
  auto dyv = [&](int m, int d) -> float {
    if constexpr (sizeof(T) == 2) return mm_widen<F>(*reinterpret_cast<const uint16_t*>(dtile + m * DS + d * 2));
    else return *reinterpret_cast<const float*>(dtile + m * DS + d * 4);
  };
  float sg[(kLnTMaxD + 255) / 256] = {0}, sb[(kLnTMaxD + 255) / 256] = {0};  // this thread's d: partial dgamma / dbeta
  for (int64_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
    const int64_t m0 = t * L::MT;
    __syncthreads();  // the previous tile is no longer read
    lnt_load_tile<T>(tile, xt, M, D, m0, tid);
    for (int idx = tid; idx < L::MT * vpr; idx += 256) {
      const int r = idx / vpr, v = idx % vpr;
      uint4 val = make_uint4(0, 0, 0, 0);
      if (m0 + r < M) val = *reinterpret_cast<const uint4*>(dy + (m0 + r) * D + v * L::EPV);
      uint32_t* p = reinterpret_cast<uint32_t*>(dtile + r * DS + v * 16);
      p[0] = val.x; p[1] = val.y; p[2] = val.z; p[3] = val.w;
    }
    if (tid < L::MT) {
      const bool ok = m0 + tid < M;
      smean[tid] = ok ? mean[m0 + tid] : 0.f;
      srstd[tid] = ok ? rstd[m0 + tid] : 0.f;
    }
    __syncthreads();
    const int m = tid % L::MT, g = tid / L::MT;
    {
      const float mu = smean[m], rs = srstd[m];
      float s1 = 0, s2 = 0;
      for (int d = g; d < D; d += L::G) {
        const float xh = (lnt_tile<T>(tile, d, m) - mu) * rs;
        const float gg = dyv(m, d) * sgam[d];
        s1 += gg;
        s2 += gg * xh;
      }
      red1[g][m] = s1;
      red2[g][m] = s2;
    }
    __syncthreads();
    if (tid < L::MT) {
      float a = 0, b = 0;
#pragma unroll
      for (int k = 0; k < L::G; ++k) { a += red1[k][tid]; b += red2[k][tid]; }
      c1[tid] = a / D;
      c2[tid] = b / D;
    }
    __syncthreads();
    // dx_t[d][m]: 4-byte stores along m
    {
      constexpr int MP = L::MT / PW;  // stores per d row
      const int mp = tid % MP, dg = tid / MP;
      const int64_t mg = m0 + mp * PW;
      if (mg < M) {
        float rs[PW], mu[PW], k1[PW], k2[PW];
#pragma unroll
        for (int e = 0; e < PW; ++e) {
          rs[e] = srstd[mp * PW + e]; mu[e] = smean[mp * PW + e]; k1[e] = c1[mp * PW + e]; k2[e] = c2[mp * PW + e];
        }
#pragma unroll 4
        for (int d = dg; d < D; d += 256 / MP) {
          const float gmm = sgam[d];
          float o[PW];
#pragma unroll
          for (int e = 0; e < PW; ++e) {
            const int mm = mp * PW + e;
            const float xh = (lnt_tile<T>(tile, d, mm) - mu[e]) * rs[e];
            o[e] = rs[e] * (dyv(mm, d) * gmm - k1[e] - xh * k2[e]);
          }
          uint32_t w;
          if constexpr (sizeof(T) == 2) w = pack16<F>(o[0], o[1]);
          else w = __float_as_uint(o[0]);
          *reinterpret_cast<uint32_t*>(dxt + static_cast<int64_t>(d) * M + mg) = w;
        }
      }
    }
    if (need_affine) {
#pragma unroll
      for (int q = 0; q < (kLnTMaxD + 255) / 256; ++q) {
        const int d = tid + q * 256;
        if (d < D) {
          for (int mm = 0; mm < L::MT; ++mm) {  // rows beyond M hold zeros in the dy tile
            const float v = dyv(mm, d);
            sg[q] += v * (lnt_tile<T>(tile, d, mm) - smean[mm]) * srstd[mm];
            sb[q] += v;
          }
        }
      }
    }
  }
  if (need_affine) {
#pragma unroll
    for (int q = 0; q < (kLnTMaxD + 255) / 256; ++q) {
      const int d = tid + q * 256;
      if (d < D) {
        part[static_cast<int64_t>(blockIdx.x) * D + d] = sg[q];
        part[(static_cast<int64_t>(gridDim.x) + blockIdx.x) * D + d] = sb[q];
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// The same two kernels for 2-byte types and D = 64 or 128 without a block-wide step: a wavefront takes 64 consecutive
// m (128-byte pieces of the rows of x_t); lane (cp, dh) owns the column pair (2 cp, 2 cp + 1) for the half dh of d and
// reads x_t as one dword per d (two whole lines per instruction, addressed as a base that is the same for all lanes +
// a 32-bit lane offset that also carries the distance between the halves).  The statistics are sums over a lane's own
// registers completed by one exchange between the lane halves.  Rows of y (forward) and of dy (backward) pass through a
// staging tile private to the wavefront, so global memory sees whole 256-byte rows; dx_t leaves as dwords, 128
// contiguous bytes per d.  Staging rows are stored pair-member-major (row 32 j + cp for column 2 cp + j): 16-byte
// accesses of consecutive lanes fall into distinct banks.  The forward keeps a second tile in flight.  The backward
// here computes the gradient of the tensor only; with the affine gradients asked for the kernel above runs.
// ------------------------------------------------------------------------------------------------
template <typename V>
__device__ __forceinline__ void store_global(char* uniform_base, uint32_t lane_offset, V value) {
  typedef __attribute__((address_space(1))) V* gptr;
  *reinterpret_cast<gptr>(reinterpret_cast<uint64_t>(uniform_base) + lane_offset) = value;
}

template <typename V>
__device__ __forceinline__ V load_global_stream(const char* uniform_base, uint32_t lane_offset) {
  typedef const __attribute__((address_space(1))) V* gptr;
  return __builtin_nontemporal_load(reinterpret_cast<gptr>(reinterpret_cast<uint64_t>(uniform_base) + lane_offset));
}

template <int D>
struct LnCols {
  static constexpr int H = D / 2;           // values of d per lane
  static constexpr int RS = 2 * D + 16;     // bytes between staged rows
  static constexpr int WAVE_LDS = 64 * RS;  // 64 rows (columns m of the tile)
};

// the H dwords of lane (cp, dh) for the tile at column m0 (which every lane of the wavefront shares); LAST: nothing reads
// x_t after this kernel (the backward: marked as a stream 45 instead of 47 us; in the forward, which reads what the
// contraction has just written, the mark costs 9 us)
template <int D, bool LAST = false, typename F>
__device__ __forceinline__ void lncols_request(uint32_t (&xv)[D / 2], const F* xt, int64_t m0, int64_t row_bytes, uint32_t voff) {
  // (one scalar base that walks down the rows; the scheduling barriers keep every address next to its load - computed
  // all at once, the D / 2 bases would not fit the scalar registers)
  const char* src = uniform_ptr(xt + m0);
#pragma unroll
  for (int i = 0; i < D / 2; ++i) {
    xv[i] = LAST ? load_global_stream<uint32_t>(src, voff) : load_global<uint32_t>(src, voff);
    src += row_bytes;
    __builtin_amdgcn_sched_barrier(0);
  }
}

template <typename F, int D>
__global__ void __launch_bounds__(256, 2) ln_t_fwd_cols_kernel(const F* __restrict__ xt, const F* __restrict__ gamma,
                                                               const F* __restrict__ beta, F* __restrict__ y, float* __restrict__ mean,
                                                               float* __restrict__ rstd, int64_t M, float eps) {
  using L = LnCols<D>;
  constexpr int H = L::H, RS = L::RS;
  extern __shared__ __align__(16) char lntc_dyn[];  // 4 wavefronts x WAVE_LDS
  __shared__ __align__(16) float sgam[D], sbet[D];
  const int tid = threadIdx.x, lane = tid & 63, cp = lane & 31, dh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  if (tid < D) {
    sgam[tid] = gamma ? tri_load(gamma, tid) : 1.0f;
    sbet[tid] = beta ? tri_load(beta, tid) : 0.0f;
  }
  __syncthreads();
  char* stage = lntc_dyn + wave * L::WAVE_LDS;
  const int64_t ntiles = (M + 63) / 64;
  const int64_t nw = static_cast<int64_t>(gridDim.x) * 4;
  const int64_t row_bytes = 2 * M;
  const float* gam = sgam + dh * H;
  const float* bet = sbet + dh * H;
  // columns past M (only in the last tile; M is even, so a pair is in or out as a whole) read the tile's first pair
  auto lane_offset = [&](int64_t tile) -> uint32_t {
    return static_cast<uint32_t>(dh * (H * row_bytes)) + (tile * 64 + 2 * cp < M ? 4u * cp : 0u);
  };
  auto work = [&](const uint32_t (&xv)[H], int64_t tile) {
    asm volatile("" ::: "memory");  // gamma / beta are read from LDS again for every tile, not kept in 2 D registers
    const int64_t m0 = tile * 64;
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int i = 0; i < H; ++i) { s0 += lo16<F>(xv[i]); s1 += hi16<F>(xv[i]); }
    s0 += __shfl_xor(s0, 32, 64);
    s1 += __shfl_xor(s1, 32, 64);
    const float mu0 = s0 * (1.0f / D), mu1 = s1 * (1.0f / D);
    float q0 = 0.f, q1 = 0.f;
#pragma unroll
    for (int i = 0; i < H; ++i) {
      const uint32_t w = again(xv[i]);
      const float c0 = lo16<F>(w) - mu0, c1 = hi16<F>(w) - mu1;
      q0 = fmaf(c0, c0, q0);
      q1 = fmaf(c1, c1, q1);
    }
    q0 += __shfl_xor(q0, 32, 64);
    q1 += __shfl_xor(q1, 32, 64);
    const float r0 = rsqrtf(q0 * (1.0f / D) + eps), r1 = rsqrtf(q1 * (1.0f / D) + eps);
    if (dh == 0 && m0 + 2 * cp < M) {
      *reinterpret_cast<float2*>(mean + m0 + 2 * cp) = make_float2(mu0, mu1);
      *reinterpret_cast<float2*>(rstd + m0 + 2 * cp) = make_float2(r0, r1);
    }
#pragma unroll
    for (int p = 0; p < H / 8; ++p) {
      uint32_t w0[4], w1[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int i = p * 8 + 2 * e;
        const float ga = gam[i], gb = gam[i + 1], ba = bet[i], bb = bet[i + 1];
        const uint32_t xa_ = again(xv[i]), xb_ = again(xv[i + 1]);
        w0[e] = pack16<F>((lo16<F>(xa_) - mu0) * r0 * ga + ba, (lo16<F>(xb_) - mu0) * r0 * gb + bb);
        w1[e] = pack16<F>((hi16<F>(xa_) - mu1) * r1 * ga + ba, (hi16<F>(xb_) - mu1) * r1 * gb + bb);
      }
      *reinterpret_cast<uint4*>(stage + cp * RS + dh * D + p * 16) = make_uint4(w0[0], w0[1], w0[2], w0[3]);
      *reinterpret_cast<uint4*>(stage + (32 + cp) * RS + dh * D + p * 16) = make_uint4(w1[0], w1[1], w1[2], w1[3]);
      __builtin_amdgcn_sched_barrier(0);  // one group of eight d at a time: its gamma / beta values die here
    }
    char* dst = const_cast<char*>(uniform_ptr(y + m0 * D));
#pragma unroll
    for (int i = 0; i < D / 8; ++i) {  // 64 rows of D / 8 vectors
      const int idx = lane + 64 * i;
      const int r = idx / (D / 8), v = idx % (D / 8);
      const int mm = 2 * (r & 31) + (r >> 5);
      if (m0 + mm < M) {
        const uint4 val = *reinterpret_cast<const uint4*>(stage + r * RS + v * 16);
        store_global<u32x4_t>(dst, static_cast<uint32_t>(mm * (2 * D) + v * 16), u32x4_t{val.x, val.y, val.z, val.w});
      }
    }
  };
  // two register sets: while one tile is worked on, the next one's rows are in flight (the loop body is two tiles
  // without a branch in between)
  int64_t tile = static_cast<int64_t>(blockIdx.x) * 4 + wave;
  if (tile >= ntiles) return;
  const int64_t mine = (ntiles - tile + nw - 1) / nw;
  uint32_t xa[H], xb[H];
  auto clamp = [&](int64_t t) { return t < ntiles ? t : ntiles - 1; };  // past the end: the last tile again, not used
  lncols_request<D>(xa, xt, clamp(tile) * 64, row_bytes, lane_offset(clamp(tile)));
  lncols_request<D>(xb, xt, clamp(tile + nw) * 64, row_bytes, lane_offset(clamp(tile + nw)));
  for (int64_t it = 0; it < mine / 2; ++it) {
    work(xa, tile);
    lncols_request<D>(xa, xt, clamp(tile + 2 * nw) * 64, row_bytes, lane_offset(clamp(tile + 2 * nw)));
    __builtin_amdgcn_sched_barrier(0);
    work(xb, tile + nw);
    lncols_request<D>(xb, xt, clamp(tile + 3 * nw) * 64, row_bytes, lane_offset(clamp(tile + 3 * nw)));
    __builtin_amdgcn_sched_barrier(0);
    tile += 2 * nw;
  }
  if (mine % 2) work(xa, tile);
}

template <typename F, int D>
__global__ void __launch_bounds__(256, 2) ln_t_bwd_cols_kernel(const F* __restrict__ dy, const F* __restrict__ xt,
                                                               const float* __restrict__ mean, const float* __restrict__ rstd,
                                                               const F* __restrict__ gamma, F* __restrict__ dxt, int64_t M) {
  using L = LnCols<D>;
  constexpr int H = L::H, RS = L::RS;
  extern __shared__ __align__(16) char lntc_dyn[];  // 4 wavefronts x WAVE_LDS
  __shared__ __align__(16) float sgam[D];
  const int tid = threadIdx.x, lane = tid & 63, cp = lane & 31, dh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  if (tid < D) sgam[tid] = gamma ? tri_load(gamma, tid) : 1.0f;
  __syncthreads();
  char* stage = lntc_dyn + wave * L::WAVE_LDS;
  const int64_t ntiles = (M + 63) / 64;
  const int64_t nw = static_cast<int64_t>(gridDim.x) * 4;
  const int64_t row_bytes = 2 * M;
  const float* gam = sgam + dh * H;
  for (int64_t tile = static_cast<int64_t>(blockIdx.x) * 4 + wave; tile < ntiles; tile += nw) {
    asm volatile("" ::: "memory");  // gamma is read from LDS again for every tile, not kept in D registers
    const int64_t m0 = tile * 64;
    const bool ok = m0 + 2 * cp < M;
    const uint32_t voff = static_cast<uint32_t>(dh * (H * row_bytes)) + (ok ? 4u * cp : 0u);
    uint32_t xv[H];
    lncols_request<D, true>(xv, xt, m0, row_bytes, voff);
    // the 64 rows of dy as they lie (D / 8 lanes per row) into the staging tile
    {
      const char* src = uniform_ptr(dy + m0 * D);
      uint4 raw[D / 8];
#pragma unroll
      for (int i = 0; i < D / 8; ++i) {
        const int idx = lane + 64 * i;
        const int r = idx / (D / 8), v = idx % (D / 8);
        const int rr = m0 + r < M ? r : 0;  // rows past the end: the tile's first row again, not used
        raw[i] = load_global<uint4>(src, static_cast<uint32_t>(rr * (2 * D) + v * 16));
      }
      __builtin_amdgcn_sched_barrier(0);  // all requests first
#pragma unroll
      for (int i = 0; i < D / 8; ++i) {
        const int idx = lane + 64 * i;
        const int r = idx / (D / 8), v = idx % (D / 8);
        *reinterpret_cast<uint4*>(stage + ((r & 1) * 32 + (r >> 1)) * RS + v * 16) = raw[i];
      }
    }
    const float2 mu = ok ? *reinterpret_cast<const float2*>(mean + m0 + 2 * cp) : make_float2(0.f, 0.f);
    const float2 rs = ok ? *reinterpret_cast<const float2*>(rstd + m0 + 2 * cp) : make_float2(0.f, 0.f);
    uint4 dv[2][H / 8];  // this lane's half of its two dy rows, packed along d
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int p = 0; p < H / 8; ++p) dv[j][p] = *reinterpret_cast<const uint4*>(stage + (j * 32 + cp) * RS + dh * D + p * 16);
    auto dy_at = [&](int j, int i) -> float {  // value i of the lane's half
      const uint4 q = dv[j][i >> 3];
      const uint32_t w = ((i >> 1) & 3) == 0 ? q.x : ((i >> 1) & 3) == 1 ? q.y : ((i >> 1) & 3) == 2 ? q.z : q.w;
      return (i & 1) ? hi16<F>(w) : lo16<F>(w);
    };
    auto dy_at2 = [&](int j, int i) -> float {  // the same for the second pass
      const uint4 q = dv[j][i >> 3];
      const uint32_t w = again(((i >> 1) & 3) == 0 ? q.x : ((i >> 1) & 3) == 1 ? q.y : ((i >> 1) & 3) == 2 ? q.z : q.w);
      return (i & 1) ? hi16<F>(w) : lo16<F>(w);
    };
    float a0 = 0.f, a1 = 0.f, b0 = 0.f, b1 = 0.f;
#pragma unroll
    for (int i = 0; i < H; ++i) {
      const float g = gam[i];
      const float g0 = dy_at(0, i) * g, g1 = dy_at(1, i) * g;
      a0 += g0;
      a1 += g1;
      b0 = fmaf(g0, (lo16<F>(xv[i]) - mu.x) * rs.x, b0);
      b1 = fmaf(g1, (hi16<F>(xv[i]) - mu.y) * rs.y, b1);
      if (i % 8 == 7) __builtin_amdgcn_sched_barrier(0);
    }
    a0 += __shfl_xor(a0, 32, 64);
    a1 += __shfl_xor(a1, 32, 64);
    b0 += __shfl_xor(b0, 32, 64);
    b1 += __shfl_xor(b1, 32, 64);
    const float k10 = a0 * (1.0f / D), k11 = a1 * (1.0f / D), k20 = b0 * (1.0f / D), k21 = b1 * (1.0f / D);
    if (ok) {
      char* dst = const_cast<char*>(uniform_ptr(dxt + m0));
#pragma unroll
      for (int i = 0; i < H; ++i) {
        const float g = gam[i];
        const uint32_t w = again(xv[i]);
        const float xh0 = (lo16<F>(w) - mu.x) * rs.x, xh1 = (hi16<F>(w) - mu.y) * rs.y;
        const float o0 = rs.x * (dy_at2(0, i) * g - k10 - xh0 * k20), o1 = rs.y * (dy_at2(1, i) * g - k11 - xh1 * k21);
        store_global<uint32_t>(dst, voff, pack16<F>(o0, o1));
        dst += row_bytes;
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// gate: out[r][c] = sigmoid(u + bu) * (v + bv) * mask;  biases and mask are indexed by row (axis 0) or column (axis 1)
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256) gate_fwd_kernel(const float* __restrict__ u, const float* __restrict__ v, const T* __restrict__ bu,
                                                       const T* __restrict__ bv, int bias_axis, const T* __restrict__ mask, int mask_axis,
                                                       T* __restrict__ out, int64_t R, int64_t Ccols) {
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tid >= R * Ccols) return;
  const int64_t r = tid / Ccols, cc = tid - r * Ccols;
  const int64_t ib = bias_axis == 0 ? r : cc;
  const float uu = u[tid] + (bu ? tri_load(bu, ib) : 0.f);
  const float vv = v[tid] + (bv ? tri_load(bv, ib) : 0.f);
  float o = vv / (1.0f + __expf(-uu));
  if (mask) o *= tri_load(mask, mask_axis == 0 ? r : cc);
  tri_store(out, tid, o);
}

// du = dout * mask * (v + bv) * s * (1 - s),  dv = dout * mask * s,  s = sigmoid(u + bu)
template <typename T>
__global__ void __launch_bounds__(256) gate_bwd_kernel(const T* __restrict__ dout, const float* __restrict__ u, const float* __restrict__ v,
                                                       const T* __restrict__ bu, const T* __restrict__ bv, int bias_axis,
                                                       const T* __restrict__ mask, int mask_axis, T* __restrict__ du, T* __restrict__ dv,
                                                       int64_t R, int64_t Ccols) {
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tid >= R * Ccols) return;
  const int64_t r = tid / Ccols, cc = tid - r * Ccols;
  const int64_t ib = bias_axis == 0 ? r : cc;
  const float uu = u[tid] + (bu ? tri_load(bu, ib) : 0.f);
  const float vv = v[tid] + (bv ? tri_load(bv, ib) : 0.f);
  const float s = 1.0f / (1.0f + __expf(-uu));
  float d = tri_load(dout, tid);
  if (mask) d *= tri_load(mask, mask_axis == 0 ? r : cc);
  tri_store(du, tid, d * vv * s * (1.0f - s));
  tri_store(dv, tid, d * s);
}

// ------------------------------------------------------------------------------------------------
// reductions of an (R x C) array: sum over columns -> [R] (one wavefront per row);
// sum over rows -> [C] (two stages through per-block partials)
// ------------------------------------------------------------------------------------------------
template <typename TI>
__global__ void __launch_bounds__(256) sum_cols_kernel(const TI* __restrict__ in, float* __restrict__ out, int64_t R, int64_t Ccols) {
  const int lane = threadIdx.x & 63;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (row >= R) return;
  float s = 0;
  for (int64_t cc = lane; cc < Ccols; cc += 64) s += tri_load(in, row * Ccols + cc);
  s = wave_sum(s);
  if (lane == 0) out[row] = s;
}

template <typename TI>
__global__ void __launch_bounds__(256) sum_rows_partial_kernel(const TI* __restrict__ in, float* __restrict__ part, int64_t R, int64_t Ccols,
                                                               int64_t rows_per_block) {
  const int64_t cc = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (cc >= Ccols) return;
  const int64_t r0 = blockIdx.y * rows_per_block, r1 = min(r0 + rows_per_block, R);
  float s = 0;
  int64_t r = r0;
  for (; r + 4 <= r1; r += 4) {  // four loads in flight, added in row order
    const float v0 = tri_load(in, r * Ccols + cc), v1 = tri_load(in, (r + 1) * Ccols + cc);
    const float v2 = tri_load(in, (r + 2) * Ccols + cc), v3 = tri_load(in, (r + 3) * Ccols + cc);
    s += v0; s += v1; s += v2; s += v3;
  }
  for (; r < r1; ++r) s += tri_load(in, r * Ccols + cc);
  part[static_cast<int64_t>(blockIdx.y) * Ccols + cc] = s;
}

// out[c] = sum_r in[r][c] in one launch for a moderate number of rows: 64 columns x 16 row lanes per block, every lane
// adds rows r = lane, lane + 16, ... in order, the 16 partial sums are added in lane order (fixed, reproducible)
template <typename TI>
__global__ void __launch_bounds__(1024) sum_rows_lds_kernel(const TI* __restrict__ in, float* __restrict__ out, int64_t R, int64_t Ccols) {
  __shared__ float s_acc[16][64];
  const int cl = threadIdx.x & 63, rl = threadIdx.x >> 6;
  const int64_t cc = static_cast<int64_t>(blockIdx.x) * 64 + cl;
  float s = 0;
  if (cc < Ccols) {
    int64_t r = rl;
    for (; r + 48 < R; r += 64) {  // four loads in flight
      const float v0 = tri_load(in, r * Ccols + cc), v1 = tri_load(in, (r + 16) * Ccols + cc);
      const float v2 = tri_load(in, (r + 32) * Ccols + cc), v3 = tri_load(in, (r + 48) * Ccols + cc);
      s += v0; s += v1; s += v2; s += v3;
    }
    for (; r < R; r += 16) s += tri_load(in, r * Ccols + cc);
  }
  s_acc[rl][cl] = s;
  __syncthreads();
  if (rl == 0 && cc < Ccols) {
    float total = 0;
#pragma unroll
    for (int t = 0; t < 16; ++t) total += s_acc[t][cl];
    out[cc] = total;
  }
}

template <typename TO>
__global__ void __launch_bounds__(256) fold_partials_kernel(const float* __restrict__ part, TO* __restrict__ out, int64_t nparts, int64_t n,
                                                            int accumulate) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= n) return;
  float s = 0;
  for (int64_t p = 0; p < nparts; ++p) s += part[p * n + i];
  if (accumulate) s += tri_load(out, i);
  tri_store(out, i, s);
}

static bool is_io(int dt) { return dt == CUEQ_F32 || dt == CUEQ_BF16 || dt == CUEQ_F16; }
// rows one launch takes when its row tiles sit on grid.y (65535 tiles of 128; a multiple of every tile height used)
constexpr int64_t kRowSlab = 65280ll * 128;

}  // namespace cueq

using namespace cueq;

// 2-byte element types: uint16_t = bfloat16 as its bits, f16bits = half as its bits
#define TRI_DISPATCH(dt, CALL_F32, CALL_BF16, CALL_F16)      \
  do {                                             \
    if ((dt) == CUEQ_F32) { CALL_F32; } else if ((dt) == CUEQ_F16) { CALL_F16; } else { CALL_BF16; } \
  } while (0)

extern "C" int cueq_gemm(int32_t in_dtype, int32_t out_dtype, int32_t trans_a, int32_t trans_b, int64_t M, int64_t N, int64_t K,
                         const void* A, int64_t lda, int64_t stride_a, const void* B, int64_t ldb, int64_t stride_b, void* C,
                         int64_t ldc, int64_t stride_c, int64_t batch, double alpha, int32_t accumulate, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(is_io(in_dtype) && is_io(out_dtype), CUEQ_ERR_UNSUPPORTED, "gemm: dtypes must be float32, bfloat16 or half");
  CUEQ_REQUIRE(in_dtype == out_dtype || in_dtype == CUEQ_F32 || out_dtype == CUEQ_F32, CUEQ_ERR_UNSUPPORTED, "gemm: bfloat16 and half do not mix");
  CUEQ_REQUIRE(M >= 0 && N >= 0 && K >= 0 && batch >= 0, CUEQ_ERR_INVALID, "gemm: negative extent");
  if (M == 0 || N == 0 || batch == 0) return CUEQ_OK;
  CUEQ_REQUIRE(A && B && C, CUEQ_ERR_INVALID, "gemm: null operand");
  if (batch > 65535) {  // grid.z holds at most 65535 batch items
    const int64_t es_in = in_dtype == CUEQ_F32 ? 4 : 2, es_out = out_dtype == CUEQ_F32 ? 4 : 2;
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {
      const int64_t bb = batch - b0 < 65535 ? batch - b0 : 65535;
      const int rc = cueq_gemm(in_dtype, out_dtype, trans_a, trans_b, M, N, K, static_cast<const char*>(A) + b0 * stride_a * es_in, lda, stride_a,
                               static_cast<const char*>(B) + b0 * stride_b * es_in, ldb, stride_b, static_cast<char*>(C) + b0 * stride_c * es_out, ldc,
                               stride_c, bb, alpha, accumulate, stream_);
      if (rc != CUEQ_OK) return rc;
    }
    return CUEQ_OK;
  }
  if (M > kRowSlab) {  // grid.y holds at most 65535 row tiles: more rows go in slabs, which are independent
    const int64_t es_in = in_dtype == CUEQ_F32 ? 4 : 2, es_out = out_dtype == CUEQ_F32 ? 4 : 2;
    for (int64_t r0 = 0; r0 < M; r0 += kRowSlab) {
      const int64_t mm = M - r0 < kRowSlab ? M - r0 : kRowSlab;
      const int rc = cueq_gemm(in_dtype, out_dtype, trans_a, trans_b, mm, N, K, static_cast<const char*>(A) + (trans_a ? r0 : r0 * lda) * es_in, lda,
                               stride_a, B, ldb, stride_b, static_cast<char*>(C) + r0 * ldc * es_out, ldc, stride_c, batch, alpha, accumulate, stream_);
      if (rc != CUEQ_OK) return rc;
    }
    return CUEQ_OK;
  }
  CUEQ_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31) && batch < 65536, CUEQ_ERR_TOO_LARGE, "gemm: extent too large");
  const int epv = in_dtype == CUEQ_F32 ? 4 : 8;
  // vectors run along k for a contraction-contiguous operand, along its other extent for a contraction-major one
  const bool aligned = K > 0 && (trans_a ? M : K) % epv == 0 && (trans_b ? N : K) % epv == 0 && lda % epv == 0 && ldb % epv == 0 &&
                       stride_a % epv == 0 && stride_b % epv == 0 && reinterpret_cast<uintptr_t>(A) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(B) % 16 == 0;
  const float al = static_cast<float>(alpha);
  const int m = static_cast<int>(M), n = static_cast<int>(N), k = static_cast<int>(K);
  const bool mixed = in_dtype != out_dtype;
  const bool mixed_ok = !mixed || (!trans_a && !trans_b) || (in_dtype != CUEQ_F32 && out_dtype == CUEQ_F32 && !trans_a && trans_b);
  if (aligned && mixed_ok) {
    const dim3 grid(static_cast<unsigned>((N + kTile - 1) / kTile), static_cast<unsigned>((M + kTile - 1) / kTile), static_cast<unsigned>(batch));
    CUEQ_REQUIRE(grid.y < 65536, CUEQ_ERR_TOO_LARGE, "gemm: too many row tiles (M <= 8388480)");
    const int64_t out_es = out_dtype == CUEQ_F32 ? 4 : 2;
    const int vec_out = (reinterpret_cast<uintptr_t>(C) % 16 == 0 && (ldc * out_es) % 16 == 0 && (stride_c * out_es) % 16 == 0) ? 1 : 0;
    // 256 x 256 tiles when both extents are multiples of 256 and there are enough of them to fill the chip
    const bool big = !mixed && M % 256 == 0 && N % 256 == 0 && (M / 256) * (N / 256) * batch >= 2 * static_cast<int64_t>(device_cus());
    // (the timing label names the tile size, so a test can tell which kernel a shape ran on)
    KernelTimer timer(in_dtype == CUEQ_F32 ? (big ? "gemm_nt_f32_256" : "gemm_nt_f32") : in_dtype == CUEQ_F16 ? (big ? "gemm_nt_f16_256" : "gemm_nt_f16") : (big ? "gemm_nt_bf16_256" : "gemm_nt_bf16"), stream);
    const dim3 grid_big(static_cast<unsigned>(N / 256), static_cast<unsigned>(M / 256), static_cast<unsigned>(batch));
#define GEMM_ARGS(TI, TO) static_cast<const TI*>(A), lda, stride_a, static_cast<const TI*>(B), ldb, stride_b, static_cast<TO*>(C), ldc, stride_c, m, n, k, al, accumulate, vec_out, 0, 1, 0, 0, 0, nullptr, 0, 0, 0, 0
#define GEMM_LAUNCH(TI, TO, TA, TB) hipLaunchKernelGGL((gemm_kernel<TI, TO, TA, TB>), grid, dim3(256), 0, stream, GEMM_ARGS(TI, TO))
#define GEMM_SZ(TI, TA, TB) do { if (big) hipLaunchKernelGGL((gemm_kernel<TI, TI, TA, TB, 4, 4, (sizeof(TI) == 2 ? 128 : 64)>), grid_big, dim3(1024), 0, stream, GEMM_ARGS(TI, TI)); else GEMM_LAUNCH(TI, TI, TA, TB); } while (0)
#define GEMM_TR(TI) do { if (trans_a && trans_b) GEMM_SZ(TI, true, true); else if (trans_a) GEMM_SZ(TI, true, false); else if (trans_b) GEMM_SZ(TI, false, true); else GEMM_SZ(TI, false, false); } while (0)
    if (in_dtype == CUEQ_F32 && out_dtype == CUEQ_F32) GEMM_TR(float);
    else if (in_dtype == CUEQ_F32 && out_dtype == CUEQ_F16) GEMM_LAUNCH(float, f16bits, false, false);
    else if (in_dtype == CUEQ_F32) GEMM_LAUNCH(float, uint16_t, false, false);
    else if (in_dtype == CUEQ_F16 && out_dtype == CUEQ_F32) { if (trans_b) GEMM_LAUNCH(f16bits, float, false, true); else GEMM_LAUNCH(f16bits, float, false, false); }
    else if (out_dtype == CUEQ_F32) { if (trans_b) GEMM_LAUNCH(uint16_t, float, false, true); else GEMM_LAUNCH(uint16_t, float, false, false); }
    else if (in_dtype == CUEQ_F16) GEMM_TR(f16bits);
    else GEMM_TR(uint16_t);
#undef GEMM_TR
#undef GEMM_SZ
#undef GEMM_LAUNCH
#undef GEMM_ARGS
  } else {
    const int64_t total = M * N;
    CUEQ_REQUIRE((total + 255) / 256 < (1ll << 31), CUEQ_ERR_TOO_LARGE, "gemm: output too large for the unaligned path");
    const dim3 grid(static_cast<unsigned>((total + 255) / 256), 1, static_cast<unsigned>(batch));
    KernelTimer timer("gemm_nt_simple", stream);
    const int64_t rsa = trans_a ? 1 : lda, ksa = trans_a ? lda : 1, rsb = trans_b ? 1 : ldb, ksb = trans_b ? ldb : 1;
#define GEMM_LAUNCH(TI, TO) hipLaunchKernelGGL((gemm_simple<TI, TO>), grid, dim3(256), 0, stream, static_cast<const TI*>(A), rsa, ksa, stride_a, static_cast<const TI*>(B), rsb, ksb, stride_b, static_cast<TO*>(C), ldc, stride_c, m, n, k, al, accumulate)
    if (in_dtype == CUEQ_F32 && out_dtype == CUEQ_F32) GEMM_LAUNCH(float, float);
    else if (in_dtype == CUEQ_F32 && out_dtype == CUEQ_F16) GEMM_LAUNCH(float, f16bits);
    else if (in_dtype == CUEQ_F32) GEMM_LAUNCH(float, uint16_t);
    else if (in_dtype == CUEQ_F16 && out_dtype == CUEQ_F32) GEMM_LAUNCH(f16bits, float);
    else if (out_dtype == CUEQ_F32) GEMM_LAUNCH(uint16_t, float);
    else if (in_dtype == CUEQ_F16) GEMM_LAUNCH(f16bits, f16bits);
    else GEMM_LAUNCH(uint16_t, uint16_t);
#undef GEMM_LAUNCH
  }
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

extern "C" int cueq_gemm_nt(int32_t in_dtype, int32_t out_dtype, int64_t M, int64_t N, int64_t K, const void* A, int64_t lda,
                            int64_t stride_a, const void* B, int64_t ldb, int64_t stride_b, void* C, int64_t ldc, int64_t stride_c,
                            int64_t batch, double alpha, int32_t accumulate, void* stream_) {
  return cueq_gemm(in_dtype, out_dtype, 0, 0, M, N, K, A, lda, stride_a, B, ldb, stride_b, C, ldc, stride_c, batch, alpha, accumulate, stream_);
}

extern "C" int cueq_gemm_table(int32_t in_dtype, int32_t out_dtype, int32_t trans_a, int32_t trans_b, int64_t M, int64_t N, int64_t K,
                               const void* A, int64_t lda, const void* B, int64_t ldb, void* C, int64_t ldc, const int64_t* table,
                               int64_t nparts, int64_t k_chunks, int64_t chunk_stride_c, double alpha, int32_t accumulate, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(is_io(in_dtype) && (out_dtype == in_dtype || out_dtype == CUEQ_F32), CUEQ_ERR_UNSUPPORTED,
               "gemm_table: float32, bfloat16 or half operands, result of the same type or float32");
  CUEQ_REQUIRE(M >= 0 && N >= 0 && K >= 0 && nparts >= 0 && k_chunks >= 1, CUEQ_ERR_INVALID, "gemm_table: bad extents");
  if (M == 0 || N == 0 || nparts == 0) return CUEQ_OK;
  CUEQ_REQUIRE(A && B && C && table, CUEQ_ERR_INVALID, "gemm_table: null operand");
  CUEQ_REQUIRE(k_chunks == 1 || (trans_a && trans_b), CUEQ_ERR_UNSUPPORTED, "gemm_table: the contraction is cut only for contraction-major operands");
  CUEQ_REQUIRE(!(trans_a && !trans_b), CUEQ_ERR_UNSUPPORTED, "gemm_table: A contraction-major with B contraction-contiguous is not built");
  if (M > kRowSlab) {
    const int64_t es_in = in_dtype == CUEQ_F32 ? 4 : 2, es_out = out_dtype == CUEQ_F32 ? 4 : 2;
    for (int64_t r0 = 0; r0 < M; r0 += kRowSlab) {
      const int64_t mm = M - r0 < kRowSlab ? M - r0 : kRowSlab;
      const int rc = cueq_gemm_table(in_dtype, out_dtype, trans_a, trans_b, mm, N, K, static_cast<const char*>(A) + (trans_a ? r0 : r0 * lda) * es_in, lda, B,
                                     ldb, static_cast<char*>(C) + r0 * ldc * es_out, ldc, table, nparts, k_chunks, chunk_stride_c, alpha, accumulate, stream_);
      if (rc != CUEQ_OK) return rc;
    }
    return CUEQ_OK;
  }
  CUEQ_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31) && nparts * k_chunks < 65536, CUEQ_ERR_TOO_LARGE, "gemm_table: extent too large");
  const int epv = in_dtype == CUEQ_F32 ? 4 : 8;
  // the table's offsets must keep the 16-byte alignment too: the caller builds it from segment offsets (checked there)
  const bool aligned = K > 0 && (trans_a ? M : K) % epv == 0 && (trans_b ? N : K) % epv == 0 && lda % epv == 0 && ldb % epv == 0 &&
                       reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(B) % 16 == 0;
  CUEQ_REQUIRE(aligned, CUEQ_ERR_UNSUPPORTED, "gemm_table: extents along vectors, strides and pointers must be multiples of 16 bytes");
  const int64_t kc = k_chunks == 1 ? K : (((K + k_chunks - 1) / k_chunks + 31) / 32) * 32;  // contraction per chunk
  const dim3 grid(static_cast<unsigned>((N + kTile - 1) / kTile), static_cast<unsigned>((M + kTile - 1) / kTile), static_cast<unsigned>(nparts * k_chunks));
  CUEQ_REQUIRE(grid.y < 65536, CUEQ_ERR_TOO_LARGE, "gemm_table: too many row tiles");
  const int vec_out = 0;  // the result offsets come from the device table: their alignment is not known here
  KernelTimer timer("gemm_table", stream);
  // results at most 64 columns wide take 256 x 64 tiles (4 x 1 wavefronts) instead of wasting half a 128 x 128 tile
  // and products of at most 64 x 64 with both operands contraction-major (weight gradients of small blocks) take one
  // wavefront each
  const bool skinny = N <= 64;
  const bool small = skinny && M <= 64 && trans_a && trans_b;
  const dim3 grid_s(1, static_cast<unsigned>((M + 255) / 256), static_cast<unsigned>(nparts * k_chunks));
  const dim3 grid_1(1, 1, static_cast<unsigned>(nparts * k_chunks));
#define GT_ARGS(TI, TO) static_cast<const TI*>(A), lda, k_chunks == 1 ? 0 : kc * lda, static_cast<const TI*>(B), ldb, k_chunks == 1 ? 0 : kc * ldb, static_cast<TO*>(C), ldc, chunk_stride_c, static_cast<int>(M), static_cast<int>(N), static_cast<int>(kc), static_cast<float>(alpha), accumulate, vec_out, k_chunks == 1 ? 0 : K, static_cast<int>(nparts), 0, 0, 0, table, 0, 3, 0, 0
#define GT(TI, TO, TA, TB) do { if (skinny) hipLaunchKernelGGL((gemm_kernel<TI, TO, TA, TB, 4, 1>), grid_s, dim3(256), 0, stream, GT_ARGS(TI, TO)); else hipLaunchKernelGGL((gemm_kernel<TI, TO, TA, TB>), grid, dim3(256), 0, stream, GT_ARGS(TI, TO)); } while (0)
#define GT_T(TI, TO) do { if (small) hipLaunchKernelGGL((gemm_kernel<TI, TO, true, true, 1, 1>), grid_1, dim3(64), 0, stream, GT_ARGS(TI, TO)); else if (trans_a && trans_b) GT(TI, TO, true, true); else if (trans_b) GT(TI, TO, false, true); else GT(TI, TO, false, false); } while (0)
  if (in_dtype == CUEQ_F32) GT_T(float, float);
  else if (in_dtype == CUEQ_F16) { if (out_dtype == CUEQ_F32) GT_T(f16bits, float); else GT_T(f16bits, f16bits); }
  else if (out_dtype == CUEQ_F32) GT_T(uint16_t, float);
  else GT_T(uint16_t, uint16_t);
#undef GT_T
#undef GT
#undef GT_ARGS
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

extern "C" int cueq_gemm_grouped(int32_t in_dtype, int32_t out_dtype, int32_t mode, int64_t M, int64_t N, int64_t K, const void* A, int64_t lda,
                                 int64_t stride_a, const void* B, int64_t ldb, int64_t stride_b, void* C, int64_t ldc, int64_t stride_c,
                                 int64_t batch, const int64_t* offsets, int64_t ngroups, int32_t trans_b, int64_t group_stride, double alpha,
                                 int32_t accumulate, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(is_io(in_dtype) && is_io(out_dtype), CUEQ_ERR_UNSUPPORTED, "gemm_grouped: dtypes must be float32, bfloat16 or half");
  CUEQ_REQUIRE(mode == 1 || mode == 2, CUEQ_ERR_INVALID, "gemm_grouped: mode must be 1 (rows grouped) or 2 (contraction grouped)");
  CUEQ_REQUIRE(M >= 0 && N >= 0 && K >= 0 && batch >= 1 && ngroups >= 0, CUEQ_ERR_INVALID, "gemm_grouped: bad extents");
  if (M == 0 || N == 0 || ngroups == 0) return CUEQ_OK;
  CUEQ_REQUIRE(A && B && C && offsets, CUEQ_ERR_INVALID, "gemm_grouped: null operand");
  CUEQ_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31) && batch * (mode == 2 ? ngroups : 1) < 65536 && ngroups < 65536,
               CUEQ_ERR_TOO_LARGE, "gemm_grouped: extent too large");
  const int epv = in_dtype == CUEQ_F32 ? 4 : 8;
  const float al = static_cast<float>(alpha);
  const int64_t out_es = out_dtype == CUEQ_F32 ? 4 : 2;
  const bool ptrs_ok = reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(B) % 16 == 0 && lda % epv == 0 && ldb % epv == 0 &&
                       stride_a % epv == 0 && stride_b % epv == 0 && group_stride % epv == 0;
  KernelTimer timer(mode == 1 ? "gemm_grouped_rows" : "gemm_grouped_k", stream);
  if (mode == 1) {
    // C[z, :] = alpha * A[z, :] . B_g^T for the rows z of group g; B_g = B + g * group_stride is N x K, or K x N with trans_b
    CUEQ_REQUIRE(in_dtype == out_dtype, CUEQ_ERR_UNSUPPORTED, "gemm_grouped: rows-grouped products keep the dtype");
    CUEQ_REQUIRE(ptrs_ok && K % epv == 0 && (!trans_b || N % epv == 0), CUEQ_ERR_UNSUPPORTED,
                 "gemm_grouped: extents, strides and pointers must be multiples of 16 bytes");
    const int64_t gy = (M + kTile - 1) / kTile + ngroups;
    CUEQ_REQUIRE(gy < 65536, CUEQ_ERR_TOO_LARGE, "gemm_grouped: too many row tiles");
    const dim3 grid(static_cast<unsigned>((N + kTile - 1) / kTile), static_cast<unsigned>(gy), static_cast<unsigned>(batch));
    const int vec_out = (reinterpret_cast<uintptr_t>(C) % 16 == 0 && (ldc * out_es) % 16 == 0 && (stride_c * out_es) % 16 == 0) ? 1 : 0;
#define GG(TI, TB) hipLaunchKernelGGL((gemm_kernel<TI, TI, false, TB>), grid, dim3(256), 0, stream, static_cast<const TI*>(A), lda, stride_a, static_cast<const TI*>(B), ldb, stride_b, static_cast<TI*>(C), ldc, stride_c, static_cast<int>(M), static_cast<int>(N), static_cast<int>(K), al, accumulate, vec_out, 0, 1, 0, 0, 0, offsets, static_cast<int>(ngroups), 1, group_stride, 0)
    if (in_dtype == CUEQ_F32) { if (trans_b) GG(float, true); else GG(float, false); }
    else if (in_dtype == CUEQ_F16) { if (trans_b) GG(f16bits, true); else GG(f16bits, false); }
    else { if (trans_b) GG(uint16_t, true); else GG(uint16_t, false); }
#undef GG
  } else {
    // C_g (M x N, at C + g * group_stride) (+)= alpha * sum over the rows z of group g of A[z, :M]^T B[z, :N]
    // (A, B row-major with z as rows: contraction-major operands); batch items are separate column blocks (stride_*)
    CUEQ_REQUIRE(ptrs_ok && M % epv == 0 && N % epv == 0, CUEQ_ERR_UNSUPPORTED,
                 "gemm_grouped: extents, strides and pointers must be multiples of 16 bytes");
    CUEQ_REQUIRE(in_dtype == out_dtype || out_dtype == CUEQ_F32, CUEQ_ERR_UNSUPPORTED, "gemm_grouped: the result is the input dtype or float32");
    const dim3 grid(static_cast<unsigned>((N + kTile - 1) / kTile), static_cast<unsigned>((M + kTile - 1) / kTile), static_cast<unsigned>(ngroups * batch));
#define GK(TI, TO) hipLaunchKernelGGL((gemm_kernel<TI, TO, true, true>), grid, dim3(256), 0, stream, static_cast<const TI*>(A), lda, 0, static_cast<const TI*>(B), ldb, 0, static_cast<TO*>(C), ldc, 0, static_cast<int>(M), static_cast<int>(N), 0, al, accumulate, 0, 0, static_cast<int>(batch), stride_a, stride_b, stride_c, offsets, static_cast<int>(ngroups), 2, 0, group_stride)
    if (in_dtype == CUEQ_F32) GK(float, float);
    else if (in_dtype == CUEQ_F16) { if (out_dtype == CUEQ_F32) GK(f16bits, float); else GK(f16bits, f16bits); }
    else if (out_dtype == CUEQ_F32) GK(uint16_t, float);
    else GK(uint16_t, uint16_t);
#undef GK
  }
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

// the resident-weights forward kernel: C weight rows (a multiple of 32) of K = 32, 64, 96 or 128 elements, 2-byte type
static size_t dual_gate_res_lds(int64_t C, int64_t K, bool ln) {
  return static_cast<size_t>(2 * C * (K == 128 ? 2 * K : 2 * K + 16) + 8 * C + (ln ? 8 * K : 0));
}
// by_rows: two inputs and the result M x C (16-byte row pieces); otherwise one input and the result C x M (4-byte column pairs)
static bool dual_gate_res_fits(int64_t C, int64_t M, int64_t K, const void* out, int64_t ldc, bool ln, bool by_rows) {
  const bool stores_ok = by_rows ? (ldc % 8 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0) : (M % 2 == 0 && ldc % 2 == 0 && reinterpret_cast<uintptr_t>(out) % 4 == 0);
  return K % 32 == 0 && K <= 128 && C % 32 == 0 && stores_ok && M >= 4096 && dual_gate_res_lds(C, K, ln) <= 160 * 1024;
}
static int launch_dual_gate_res(int64_t C, int64_t M, int64_t K, const void* W1, const void* W2, int64_t ldw, const void* X, const void* X2,
                                int64_t ldx, const void* bias1, const void* bias2, const void* mask, void* out, int64_t ldc, const void* gamma,
                                const void* beta, float eps, void* xhat, int64_t ldxh, float* mean, float* rstd, bool half, hipStream_t stream) {
  const bool by_rows = X2 != nullptr;
  const size_t lds = dual_gate_res_lds(C, K, xhat != nullptr);
  const int64_t ntiles = (M + (by_rows ? 31 : 63)) / (by_rows ? 32 : 64);
  int64_t gx = (ntiles + 7) / 8;
  if (gx > device_cus()) gx = device_cus();
#define DGR_F(FT, KT, LN, RW) do { auto kfn = dual_gate_res_kernel<FT, KT, LN, RW>; \
    CUEQ_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kfn), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds))); \
    hipLaunchKernelGGL(kfn, dim3(static_cast<unsigned>(gx)), dim3(512), lds, stream, static_cast<const FT*>(W1), static_cast<const FT*>(W2), ldw, static_cast<const FT*>(X), static_cast<const FT*>(X2), ldx, static_cast<const FT*>(bias1), static_cast<const FT*>(bias2), static_cast<const FT*>(mask), static_cast<FT*>(out), ldc, static_cast<int>(C), static_cast<int>(M), static_cast<const FT*>(gamma), static_cast<const FT*>(beta), eps, static_cast<FT*>(xhat), ldxh, mean, rstd); } while (0)
#define DGR(KT, LN, RW) do { if (half) DGR_F(f16bits, KT, LN, RW); else DGR_F(uint16_t, KT, LN, RW); } while (0)
#define DGR_K(LN, RW) do { switch (K / 32) { case 1: DGR(1, LN, RW); break; case 2: DGR(2, LN, RW); break; case 3: DGR(3, LN, RW); break; default: DGR(4, LN, RW); break; } } while (0)
  if (by_rows) DGR_K(false, true); else if (xhat) DGR_K(true, false); else DGR_K(false, false);
#undef DGR_K
#undef DGR
#undef DGR_F
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

extern "C" int cueq_dual_gate(int32_t dtype, int32_t backward, int64_t M, int64_t N, int64_t K, const void* A1, const void* A2, int64_t lda,
                              const void* B1, const void* B2, int64_t ldb, const void* bias1, const void* bias2, int32_t bias_axis,
                              const void* mask, int32_t mask_axis, const void* dC, void* out1, void* out2, int64_t ldc, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(is_io(dtype), CUEQ_ERR_UNSUPPORTED, "dual_gate: dtype must be float32 or bfloat16");
  CUEQ_REQUIRE(M >= 0 && N >= 0 && K > 0, CUEQ_ERR_INVALID, "dual_gate: bad extents");
  if (M == 0 || N == 0) return CUEQ_OK;
  CUEQ_REQUIRE(A1 && A2 && B1 && out1 && (!backward || (dC && out2)), CUEQ_ERR_INVALID, "dual_gate: null operand");
  const int epv = dtype == CUEQ_F32 ? 4 : 8;
  const bool aligned = K % epv == 0 && lda % epv == 0 && ldb % epv == 0 &&
                       ((reinterpret_cast<uintptr_t>(A1) | reinterpret_cast<uintptr_t>(A2) | reinterpret_cast<uintptr_t>(B1) | reinterpret_cast<uintptr_t>(B2)) & 15) == 0;
  CUEQ_REQUIRE(aligned, CUEQ_ERR_UNSUPPORTED, "dual_gate: K, row strides and pointers must be multiples of 16 bytes");
  if (M > kRowSlab) {
    const int64_t es = dtype == CUEQ_F32 ? 4 : 2;
    auto rows = [&](const void* p, int64_t ld, int64_t r0) { return p ? static_cast<const void*>(static_cast<const char*>(p) + r0 * ld * es) : nullptr; };
    for (int64_t r0 = 0; r0 < M; r0 += kRowSlab) {
      const int64_t mm = M - r0 < kRowSlab ? M - r0 : kRowSlab;
      const int rc = cueq_dual_gate(dtype, backward, mm, N, K, rows(A1, lda, r0), rows(A2, lda, r0), lda, B1, B2, ldb,
                                    bias_axis == 0 ? rows(bias1, 1, r0) : bias1, bias_axis == 0 ? rows(bias2, 1, r0) : bias2, bias_axis,
                                    mask_axis == 0 ? rows(mask, 1, r0) : mask, mask_axis, rows(dC, ldc, r0), const_cast<void*>(rows(out1, ldc, r0)),
                                    const_cast<void*>(rows(out2, ldc, r0)), ldc, stream_);
      if (rc != CUEQ_OK) return rc;
    }
    return CUEQ_OK;
  }
  const int64_t gy = (M + kTile - 1) / kTile, gx = (N + kTile - 1) / kTile;
  CUEQ_REQUIRE(gy < 65536 && gx < (1ll << 31) && M < (1ll << 31) && N < (1ll << 31), CUEQ_ERR_TOO_LARGE, "dual_gate: extent too large");
  const dim3 grid(static_cast<unsigned>(gx), static_cast<unsigned>(gy));
  const bool share = B2 == nullptr || B2 == B1;
  const int vec_out = (reinterpret_cast<uintptr_t>(out1) % 16 == 0 && ldc % epv == 0) ? 1 : 0;
  KernelTimer timer(backward ? "dual_gate_bwd" : "dual_gate_fwd", stream);
  // forward with one shared right operand, biases along the rows and the mask along the columns, in a 2-byte type:
  // the left operands (the weights, M rows) stay resident in LDS when they fit
  if (dtype != CUEQ_F32 && !backward && share && (!(bias1 || bias2) || bias_axis == 0) && (!mask || mask_axis == 1) &&
      dual_gate_res_fits(M, N, K, out1, ldc, false, false)) {
    return launch_dual_gate_res(M, N, K, A1, A2, lda, B1, nullptr, ldb, bias1, bias2, mask, out1, ldc, nullptr, nullptr, 0.f, nullptr, 0, nullptr, nullptr, dtype == CUEQ_F16, stream);
  }
  // the mirrored case - two left operands of many rows, the weights on the right, biases along the columns and the mask
  // along the rows: the same kernel with the weights (N rows) resident, two inputs and the result by rows
  if (dtype != CUEQ_F32 && !backward && !share && A2 != A1 && (!(bias1 || bias2) || bias_axis == 1) && (!mask || mask_axis == 0) && M <= kRowSlab &&
      dual_gate_res_fits(N, M, K, out1, ldc, false, true)) {
    return launch_dual_gate_res(N, M, K, B1, B2, ldb, A1, A2, lda, bias1, bias2, mask, out1, ldc, nullptr, nullptr, 0.f, nullptr, 0, nullptr, nullptr, dtype == CUEQ_F16, stream);
  }
#define DG(TI, BW, SH) hipLaunchKernelGGL((dual_gate_kernel<TI, BW, SH>), grid, dim3(512), 0, stream, static_cast<const TI*>(A1), static_cast<const TI*>(A2), lda, static_cast<const TI*>(B1), static_cast<const TI*>(B2), ldb, static_cast<const TI*>(bias1), static_cast<const TI*>(bias2), bias_axis, static_cast<const TI*>(mask), mask_axis, static_cast<const TI*>(dC), static_cast<TI*>(out1), static_cast<TI*>(out2), ldc, static_cast<int>(M), static_cast<int>(N), static_cast<int>(K), vec_out)
#define DG_T(TI) do { if (backward) { if (share) DG(TI, true, true); else DG(TI, true, false); } else { if (share) DG(TI, false, true); else DG(TI, false, false); } } while (0)
  TRI_DISPATCH(dtype, DG_T(float), DG_T(uint16_t), DG_T(f16bits));
#undef DG_T
#undef DG
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

extern "C" int cueq_ln_dual_gate(int32_t dtype, int64_t C, int64_t M, int64_t K, const void* W1, const void* W2, int64_t ldw, const void* X,
                                 int64_t ldx, const void* gamma, const void* beta, double eps, const void* bias1, const void* bias2,
                                 const void* mask, void* out, int64_t ldc, void* xhat, int64_t ldxh, float* mean, float* rstd, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(dtype == CUEQ_BF16 || dtype == CUEQ_F16, CUEQ_ERR_UNSUPPORTED, "ln_dual_gate: built for bfloat16 and half (compose cueq_layer_norm_fwd and cueq_dual_gate otherwise)");
  CUEQ_REQUIRE(C > 0 && M >= 0 && K > 0, CUEQ_ERR_INVALID, "ln_dual_gate: bad extents");
  if (M == 0) return CUEQ_OK;
  CUEQ_REQUIRE(W1 && W2 && X && out && xhat && mean && rstd, CUEQ_ERR_INVALID, "ln_dual_gate: null operand");
  const uintptr_t ptrs = reinterpret_cast<uintptr_t>(W1) | reinterpret_cast<uintptr_t>(W2) | reinterpret_cast<uintptr_t>(X) | reinterpret_cast<uintptr_t>(xhat);
  CUEQ_REQUIRE((ptrs & 15) == 0 && ldw % 8 == 0 && ldx % 8 == 0 && ldxh % 8 == 0 && ldw >= K && ldx >= K && ldxh >= K, CUEQ_ERR_UNSUPPORTED,
               "ln_dual_gate: row strides and pointers must be multiples of 16 bytes");
  CUEQ_REQUIRE(M <= kRowSlab && C < (1ll << 31) && ldc >= M, CUEQ_ERR_TOO_LARGE, "ln_dual_gate: extent too large");
  CUEQ_REQUIRE(dual_gate_res_fits(C, M, K, out, ldc, true, false), CUEQ_ERR_UNSUPPORTED,
               "ln_dual_gate: needs K = 32, 64, 96 or 128, C a multiple of 32 that fits the local data share, an even M of at least 4096 and an even ldc");
  KernelTimer timer("ln_dual_gate_fwd", stream);
  return launch_dual_gate_res(C, M, K, W1, W2, ldw, X, nullptr, ldx, bias1, bias2, mask, out, ldc, gamma, beta, static_cast<float>(eps), xhat, ldxh, mean, rstd, dtype == CUEQ_F16, stream);
}

// ln_x != NULL: the LayerNorm backward in the same kernel (cueq_gate_bwd_input_ln)
static int gate_bwd_input_impl(int32_t dtype, int64_t C, int64_t M, int64_t K, const void* W1, const void* W2, int64_t ldw,
                               const void* X1, const void* X2, int64_t ldx,
                               const void* bias1, const void* bias2, const void* mask, const void* dC, int64_t ldc,
                               int32_t dc_by_row, void* dX1, void* dX2, int64_t lddx, int32_t accumulate, void* dU, void* dV,
                               const void* ln_x, int64_t ldlx, const float* ln_mean, const float* ln_rstd, const void* ln_gamma, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(is_io(dtype), CUEQ_ERR_UNSUPPORTED, "gate_bwd_input: dtype must be float32 or bfloat16");
  CUEQ_REQUIRE(C >= 0 && M >= 0 && K > 0, CUEQ_ERR_INVALID, "gate_bwd_input: bad extents");
  if (M == 0) return CUEQ_OK;
  CUEQ_REQUIRE(K % 32 == 0 && K <= 128, CUEQ_ERR_UNSUPPORTED, "gate_bwd_input: K must be 32, 64, 96 or 128");
  CUEQ_REQUIRE(C % 32 == 0 && C > 0, CUEQ_ERR_UNSUPPORTED, "gate_bwd_input: C must be a positive multiple of 32");
  CUEQ_REQUIRE(M < (1ll << 31) - kTile && C < (1ll << 31), CUEQ_ERR_TOO_LARGE, "gate_bwd_input: extent too large");
  CUEQ_REQUIRE(W1 && W2 && X1 && dC && dX1 && (!dU == !dV), CUEQ_ERR_INVALID, "gate_bwd_input: null operand");
  const bool bf = dtype != CUEQ_F32, half = dtype == CUEQ_F16;
  const bool split = X2 != nullptr && X2 != X1;
  CUEQ_REQUIRE(!split || dX2, CUEQ_ERR_INVALID, "gate_bwd_input: two inputs need two gradients");
  CUEQ_REQUIRE(!(split && accumulate), CUEQ_ERR_UNSUPPORTED, "gate_bwd_input: accumulate needs a single input");
  const int epv = bf ? 8 : 4;
  const uintptr_t ptrs = reinterpret_cast<uintptr_t>(W1) | reinterpret_cast<uintptr_t>(W2) | reinterpret_cast<uintptr_t>(X1) | reinterpret_cast<uintptr_t>(X2) |
                         (dc_by_row ? 0 : reinterpret_cast<uintptr_t>(dC)) | reinterpret_cast<uintptr_t>(dX1) | reinterpret_cast<uintptr_t>(dX2) |
                         reinterpret_cast<uintptr_t>(dU) | reinterpret_cast<uintptr_t>(dV);
  const bool aligned = (ptrs & 15) == 0 && ldw % epv == 0 && ldx % epv == 0 && lddx % epv == 0 && (dc_by_row || ldc % epv == 0);
  CUEQ_REQUIRE(aligned, CUEQ_ERR_UNSUPPORTED, "gate_bwd_input: row strides and pointers must be multiples of 16 bytes");
  CUEQ_REQUIRE(split == !dc_by_row, CUEQ_ERR_UNSUPPORTED, "gate_bwd_input: built for one input with dC by rows (C x M) and two inputs with dC by columns (M x C)");
  const int64_t es = bf ? 2 : 4;
  if (!dc_by_row && ldc > 0 && (M * ldc + 8) * es >= (1ll << 32)) {
    // dC (M x C) is addressed with 32-bit byte offsets from a uniform base: more rows go in slabs (rows are independent)
    const int64_t slab = (((1ll << 32) / es - 8) / ldc) & ~int64_t(255);
    CUEQ_REQUIRE(slab > 0, CUEQ_ERR_TOO_LARGE, "gate_bwd_input: row stride of dC too large");
    auto rows = [&](const void* p, int64_t ld, int64_t r0) { return p ? static_cast<const void*>(static_cast<const char*>(p) + r0 * ld * es) : nullptr; };
    for (int64_t r0 = 0; r0 < M; r0 += slab) {
      const int64_t mm = M - r0 < slab ? M - r0 : slab;
      const int rc = cueq_gate_bwd_input(dtype, C, mm, K, W1, W2, ldw, rows(X1, ldx, r0), rows(X2, ldx, r0), ldx, bias1, bias2, rows(mask, 1, r0),
                                         rows(dC, ldc, r0), ldc, 0, const_cast<void*>(rows(dX1, lddx, r0)), const_cast<void*>(rows(dX2, lddx, r0)), lddx,
                                         accumulate, const_cast<void*>(rows(dU, ldc, r0)), const_cast<void*>(rows(dV, ldc, r0)), stream_);
      if (rc != CUEQ_OK) return rc;
    }
    return CUEQ_OK;
  }
  CUEQ_REQUIRE(ldc >= 0 && ldw >= 0 && 32 * ldw * es < (1ll << 31) &&
                   (dc_by_row ? (4 * ldc + M) : (M * ldc + 8)) * es < (1ll << 32),
               CUEQ_ERR_TOO_LARGE, "gate_bwd_input: strides too large for 32-bit lane offsets");
  KernelTimer timer(ln_x ? "gate_bwd_input_ln" : "gate_bwd_input", stream);
  if (bf) {
    // weights resident in LDS when they fit (2 C rows of 2 K + 16 bytes, biases, with two inputs the staging tiles)
    const int nwaves = split ? 4 : 8;
    const size_t lds = static_cast<size_t>(2 * C * (K == 128 ? 2 * K : 2 * K + 16) + 8 * C + (split ? nwaves * 8 * (2 * K + 16) : 0) + (ln_x ? 4 * K : 0));
    // (dC by rows is read, and the gate gradients written, as 4-byte column pairs)
    const bool pairs_ok = !dc_by_row || (M % 2 == 0 && ldc % 2 == 0 && reinterpret_cast<uintptr_t>(dC) % 4 == 0);
    if (lds <= 160 * 1024 && pairs_ok) {
      const int64_t ntiles = (M + 31) / 32;
      int64_t gx = (ntiles + nwaves - 1) / nwaves;
      if (gx > device_cus()) gx = device_cus();
#define GBR_F(FT, KT, SP) do { auto kfn = gate_bwd_input_res_kernel<FT, KT, SP, !SP, false>; \
        CUEQ_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kfn), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds))); \
        hipLaunchKernelGGL(kfn, dim3(static_cast<unsigned>(gx)), dim3(SP ? 256 : 512), lds, stream, static_cast<const FT*>(W1), static_cast<const FT*>(W2), ldw, static_cast<const FT*>(X1), static_cast<const FT*>(X2), ldx, static_cast<const FT*>(bias1), static_cast<const FT*>(bias2), static_cast<const FT*>(mask), static_cast<const FT*>(dC), ldc, static_cast<FT*>(dX1), static_cast<FT*>(dX2), lddx, accumulate, static_cast<FT*>(dU), static_cast<FT*>(dV), static_cast<int>(C), static_cast<int>(M), static_cast<const FT*>(nullptr), int64_t(0), static_cast<const float*>(nullptr), static_cast<const float*>(nullptr), static_cast<const FT*>(nullptr)); } while (0)
#define GBR(KT, SP) do { if (half) GBR_F(f16bits, KT, SP); else GBR_F(uint16_t, KT, SP); } while (0)
#define GBR_K(SP) do { switch (K / 32) { case 1: GBR(1, SP); break; case 2: GBR(2, SP); break; case 3: GBR(3, SP); break; default: GBR(4, SP); break; } } while (0)
#define GBL_F(FT, KT) do { auto kfn = gate_bwd_input_res_kernel<FT, KT, false, true, true>; \
        CUEQ_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kfn), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds))); \
        hipLaunchKernelGGL(kfn, dim3(static_cast<unsigned>(gx)), dim3(512), lds, stream, static_cast<const FT*>(W1), static_cast<const FT*>(W2), ldw, static_cast<const FT*>(X1), static_cast<const FT*>(X2), ldx, static_cast<const FT*>(bias1), static_cast<const FT*>(bias2), static_cast<const FT*>(mask), static_cast<const FT*>(dC), ldc, static_cast<FT*>(dX1), static_cast<FT*>(dX2), lddx, accumulate, static_cast<FT*>(dU), static_cast<FT*>(dV), static_cast<int>(C), static_cast<int>(M), static_cast<const FT*>(ln_x), ldlx, ln_mean, ln_rstd, static_cast<const FT*>(ln_gamma)); } while (0)
#define GBL(KT) do { if (half) GBL_F(f16bits, KT); else GBL_F(uint16_t, KT); } while (0)
      if (ln_x) { switch (K / 32) { case 1: GBL(1); break; case 2: GBL(2); break; case 3: GBL(3); break; default: GBL(4); break; } }
      else if (split) GBR_K(true); else GBR_K(false);
#undef GBL
#undef GBL_F
#undef GBR_K
#undef GBR
#undef GBR_F
      CUEQ_CHECK_HIP(hipGetLastError());
      return CUEQ_OK;
    }
  }
  CUEQ_REQUIRE(!ln_x, CUEQ_ERR_UNSUPPORTED, "gate_bwd_input_ln: needs bfloat16, the weights fitting the local data share, an even M and ldc (compose cueq_gate_bwd_input and cueq_layer_norm_bwd otherwise)");
#define GBI(TI, KT, SP) hipLaunchKernelGGL((gate_bwd_input_kernel<TI, KT, SP, !SP>), dim3(static_cast<unsigned>((M + gbi_threads<TI, SP>() / 2 - 1) / (gbi_threads<TI, SP>() / 2))), dim3(gbi_threads<TI, SP>()), 0, stream, static_cast<const TI*>(W1), static_cast<const TI*>(W2), ldw, static_cast<const TI*>(X1), static_cast<const TI*>(X2), ldx, static_cast<const TI*>(bias1), static_cast<const TI*>(bias2), static_cast<const TI*>(mask), static_cast<const TI*>(dC), ldc, static_cast<TI*>(dX1), static_cast<TI*>(dX2), lddx, accumulate, static_cast<TI*>(dU), static_cast<TI*>(dV), static_cast<int>(C), static_cast<int>(M))
#define GBI_K(TI, SP) do { switch (K / 32) { case 1: GBI(TI, 1, SP); break; case 2: GBI(TI, 2, SP); break; case 3: GBI(TI, 3, SP); break; default: GBI(TI, 4, SP); break; } } while (0)
#define GBI_T(TI) do { if (split) GBI_K(TI, true); else GBI_K(TI, false); } while (0)
  TRI_DISPATCH(dtype, GBI_T(float), GBI_T(uint16_t), GBI_T(f16bits));
#undef GBI_T
#undef GBI_K
#undef GBI
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

extern "C" int cueq_gate_bwd_input(int32_t dtype, int64_t C, int64_t M, int64_t K, const void* W1, const void* W2, int64_t ldw,
                                   const void* X1, const void* X2, int64_t ldx,
                                   const void* bias1, const void* bias2, const void* mask, const void* dC, int64_t ldc,
                                   int32_t dc_by_row, void* dX1, void* dX2, int64_t lddx, int32_t accumulate, void* dU, void* dV,
                                   void* stream_) {
  return gate_bwd_input_impl(dtype, C, M, K, W1, W2, ldw, X1, X2, ldx, bias1, bias2, mask, dC, ldc, dc_by_row, dX1, dX2, lddx, accumulate, dU, dV,
                             nullptr, 0, nullptr, nullptr, nullptr, stream_);
}

extern "C" int cueq_gate_bwd_input_ln(int32_t dtype, int64_t C, int64_t M, int64_t K, const void* W1, const void* W2, int64_t ldw, const void* X,
                                      int64_t ldx, const void* bias1, const void* bias2, const void* mask, const void* dC, int64_t ldc,
                                      void* dX, int64_t lddx, int32_t accumulate, const void* ln_x, int64_t ldlx, const float* ln_mean,
                                      const float* ln_rstd, const void* ln_gamma, void* stream_) {
  CUEQ_REQUIRE(dtype == CUEQ_BF16 || dtype == CUEQ_F16, CUEQ_ERR_UNSUPPORTED, "gate_bwd_input_ln: built for bfloat16 and half");
  CUEQ_REQUIRE(ln_x && ln_mean && ln_rstd, CUEQ_ERR_INVALID, "gate_bwd_input_ln: null operand");
  CUEQ_REQUIRE(reinterpret_cast<uintptr_t>(ln_x) % 16 == 0 && ldlx % 8 == 0 && ldlx >= K, CUEQ_ERR_UNSUPPORTED,
               "gate_bwd_input_ln: the LayerNorm input rows must be 16-byte aligned");
  return gate_bwd_input_impl(dtype, C, M, K, W1, W2, ldw, X, nullptr, ldx, bias1, bias2, mask, dC, ldc, 1, dX, nullptr, lddx, accumulate, nullptr, nullptr,
                             ln_x, ldlx, ln_mean, ln_rstd, ln_gamma, stream_);
}

extern "C" int64_t cueq_gemm_tn_items(int64_t rows, int32_t nparts) {
  if (nparts < 1) nparts = 1;
  int64_t chunks = static_cast<int64_t>(device_cus()) * 2 / nparts;  // at most two blocks per CU: no tail round
  const int64_t most = (rows + 4 * kTnRows - 1) / (4 * kTnRows);  // at least 64 rows per chunk
  if (chunks > most) chunks = most;
  if (chunks < 1) chunks = 1;
  return chunks * nparts;
}

extern "C" int cueq_gemm_tn(int32_t in_dtype, int64_t M, int64_t N, int64_t rows, const void* A, int64_t lda, int64_t stride_a,
                            const void* B, int64_t ldb, int64_t stride_b, int32_t nparts, float* partials, double alpha, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(is_io(in_dtype), CUEQ_ERR_UNSUPPORTED, "gemm_tn: dtype must be float32 or bfloat16");
  CUEQ_REQUIRE(M > 0 && N > 0 && rows >= 0 && nparts >= 1, CUEQ_ERR_INVALID, "gemm_tn: bad extents");
  CUEQ_REQUIRE(A && B && partials, CUEQ_ERR_INVALID, "gemm_tn: null operand");
  CUEQ_REQUIRE(M < (1ll << 20) && N < (1ll << 20), CUEQ_ERR_TOO_LARGE, "gemm_tn: result too large");
  const int64_t items = cueq_gemm_tn_items(rows, nparts);
  const int64_t chunks = items / nparts;
  const int64_t rpc = rows == 0 ? 0 : (((rows + chunks - 1) / chunks + kTnRows - 1) / kTnRows) * kTnRows;
  CUEQ_REQUIRE(items < 65536, CUEQ_ERR_TOO_LARGE, "gemm_tn: too many items");
  const dim3 grid(static_cast<unsigned>((N + kTile - 1) / kTile), static_cast<unsigned>((M + kTile - 1) / kTile), static_cast<unsigned>(items));
  const bool vec = M % 8 == 0 && N % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0 && stride_a % 8 == 0 && stride_b % 8 == 0 &&
                   reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(B) % 16 == 0;
  KernelTimer timer("gemm_tn", stream);
  if (in_dtype != CUEQ_F32 && vec && rows > 0) {
    // 2-byte inputs: MFMA on contraction-major tiles (transposing LDS reads); batch items = (row chunk, part)
    const int64_t rpc32 = (((rows + chunks - 1) / chunks + 31) / 32) * 32;
#define TN2(FT) hipLaunchKernelGGL((gemm_kernel<FT, float, true, true>), grid, dim3(256), 0, stream, static_cast<const FT*>(A), lda, \
                       rpc32 * lda, static_cast<const FT*>(B), ldb, rpc32 * ldb, partials, N, static_cast<int64_t>(M) * N, \
                       static_cast<int>(M), static_cast<int>(N), static_cast<int>(rpc32), static_cast<float>(alpha), 0, 0, rows, nparts, \
                       stride_a, stride_b, chunks * static_cast<int64_t>(M) * N, nullptr, 0, 0, 0, 0)
    if (in_dtype == CUEQ_F16) TN2(f16bits); else TN2(uint16_t);
#undef TN2
    CUEQ_CHECK_HIP(hipGetLastError());
    return CUEQ_OK;
  }
#define TN_LAUNCH(TI, V) hipLaunchKernelGGL((gemm_tn_kernel<TI, V>), grid, dim3(256), 0, stream, static_cast<const TI*>(A), lda, stride_a, static_cast<const TI*>(B), ldb, stride_b, partials, static_cast<int>(M), static_cast<int>(N), rows, rpc, nparts, static_cast<float>(alpha))
  if (in_dtype == CUEQ_F32) { if (vec) TN_LAUNCH(float, true); else TN_LAUNCH(float, false); }
  else if (in_dtype == CUEQ_F16) { if (vec) TN_LAUNCH(f16bits, true); else TN_LAUNCH(f16bits, false); }
  else { if (vec) TN_LAUNCH(uint16_t, true); else TN_LAUNCH(uint16_t, false); }
#undef TN_LAUNCH
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

extern "C" int cueq_transpose(int32_t dtype, int64_t batch, int64_t rows, int64_t cols, const void* in, void* out, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(is_io(dtype), CUEQ_ERR_UNSUPPORTED, "transpose: dtype must be float32 or bfloat16");
  if (batch <= 0 || rows <= 0 || cols <= 0) return CUEQ_OK;
  CUEQ_REQUIRE(in && out, CUEQ_ERR_INVALID, "transpose: null operand");
  CUEQ_REQUIRE(rows < (1ll << 31) && cols < (1ll << 31), CUEQ_ERR_TOO_LARGE, "transpose: extent too large");
  if (dtype != CUEQ_F32 && rows % 2 == 0 && cols % 2 == 0 && reinterpret_cast<uintptr_t>(in) % 4 == 0 && reinterpret_cast<uintptr_t>(out) % 4 == 0) {
    int64_t gy2 = (rows + 63) / 64, gx2 = (cols + 63) / 64;
    const int rows_on_x = gy2 >= 65536 ? 1 : 0;
    if (rows_on_x) { const int64_t t = gx2; gx2 = gy2; gy2 = t; }
    CUEQ_REQUIRE(gy2 < 65536 && gx2 < (1ll << 31) && batch < 65536, CUEQ_ERR_TOO_LARGE, "transpose: extent too large");
    KernelTimer timer("transpose", stream);
    hipLaunchKernelGGL(transpose16_kernel, dim3(static_cast<unsigned>(gx2), static_cast<unsigned>(gy2), static_cast<unsigned>(batch)), dim3(256), 0, stream,
                       static_cast<const uint16_t*>(in), static_cast<uint16_t*>(out), static_cast<int>(rows), static_cast<int>(cols), rows_on_x);
    CUEQ_CHECK_HIP(hipGetLastError());
    return CUEQ_OK;
  }
  int64_t gy = (rows + 31) / 32, gx = (cols + 31) / 32;
  const int rows_on_x = gy >= 65536 ? 1 : 0;
  if (rows_on_x) { const int64_t t = gx; gx = gy; gy = t; }
  CUEQ_REQUIRE(gy < 65536 && batch < 65536 && gx < (1ll << 31), CUEQ_ERR_TOO_LARGE, "transpose: extent too large");
  const dim3 grid(static_cast<unsigned>(gx), static_cast<unsigned>(gy), static_cast<unsigned>(batch));
  KernelTimer timer("transpose", stream);
  TRI_DISPATCH(dtype,
               hipLaunchKernelGGL(transpose_kernel<float>, grid, dim3(256), 0, stream, static_cast<const float*>(in), static_cast<float*>(out), static_cast<int>(rows), static_cast<int>(cols), rows_on_x),
               hipLaunchKernelGGL(transpose_kernel<uint16_t>, grid, dim3(256), 0, stream, static_cast<const uint16_t*>(in), static_cast<uint16_t*>(out), static_cast<int>(rows), static_cast<int>(cols), rows_on_x),
               hipLaunchKernelGGL(transpose_kernel<f16bits>, grid, dim3(256), 0, stream, static_cast<const f16bits*>(in), static_cast<f16bits*>(out), static_cast<int>(rows), static_cast<int>(cols), rows_on_x));
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

extern "C" int cueq_layer_norm_fwd(int32_t dtype, int64_t rows, int64_t D, const void* x, const void* gamma, const void* beta, double eps,
                                   void* y, float* mean, float* rstd, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(is_io(dtype), CUEQ_ERR_UNSUPPORTED, "layer_norm: dtype must be float32 or bfloat16");
  CUEQ_REQUIRE(D > 0 && D <= 64 * kLnMaxPerLane, CUEQ_ERR_UNSUPPORTED, "layer_norm: hidden size must be in [1, %d]", 64 * kLnMaxPerLane);
  if (rows <= 0) return CUEQ_OK;
  CUEQ_REQUIRE(x && y && mean && rstd, CUEQ_ERR_INVALID, "layer_norm: null operand");
  CUEQ_REQUIRE((rows + 3) / 4 < (1ll << 31), CUEQ_ERR_TOO_LARGE, "layer_norm: too many rows");
  const dim3 grid(static_cast<unsigned>((rows + 3) / 4));
  KernelTimer timer("layer_norm_fwd", stream);
  const bool al16 = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(gamma) | reinterpret_cast<uintptr_t>(beta)) & 15) == 0;
  if (al16 && (D == 32 || D == 64 || D == 128 || D == 256 || D == 512)) {
    const int L = static_cast<int>(D / 8);
    const int64_t rpb = 4 * (64 / L);
    const dim3 g8(static_cast<unsigned>((rows + rpb - 1) / rpb));
#define LN8(T, LL) hipLaunchKernelGGL((ln_fwd_rows8<T, LL>), g8, dim3(256), 0, stream, static_cast<const T*>(x), static_cast<const T*>(gamma), static_cast<const T*>(beta), static_cast<T*>(y), mean, rstd, rows, static_cast<float>(eps))
#define LN8_L(T) do { switch (L) { case 4: LN8(T, 4); break; case 8: LN8(T, 8); break; case 16: LN8(T, 16); break; case 32: LN8(T, 32); break; default: LN8(T, 64); } } while (0)
    TRI_DISPATCH(dtype, LN8_L(float), LN8_L(uint16_t), LN8_L(f16bits));
#undef LN8_L
#undef LN8
    CUEQ_CHECK_HIP(hipGetLastError());
    return CUEQ_OK;
  }
  const int nq = static_cast<int>((D + 63) / 64);
#define LN_FWD(T, NQ) hipLaunchKernelGGL((ln_fwd_kernel<T, NQ>), grid, dim3(256), 0, stream, static_cast<const T*>(x), static_cast<const T*>(gamma), static_cast<const T*>(beta), static_cast<T*>(y), mean, rstd, rows, static_cast<int>(D), static_cast<float>(eps))
#define LN_FWD_NQ(T) do { if (nq <= 1) LN_FWD(T, 1); else if (nq <= 2) LN_FWD(T, 2); else if (nq <= 4) LN_FWD(T, 4); else if (nq <= 8) LN_FWD(T, 8); else LN_FWD(T, 16); } while (0)
  TRI_DISPATCH(dtype, LN_FWD_NQ(float), LN_FWD_NQ(uint16_t), LN_FWD_NQ(f16bits));
#undef LN_FWD_NQ
#undef LN_FWD
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

static int64_t ln_bwd_blocks(int64_t rows) {
  int64_t nb = static_cast<int64_t>(device_cus()) * 4;
  const int64_t most = (rows + 15) / 16;
  if (nb > most) nb = most;
  return nb < 1 ? 1 : nb;
}

extern "C" int64_t cueq_layer_norm_bwd_workspace(int64_t rows, int64_t D) { return ln_bwd_blocks(rows) * 2 * D * static_cast<int64_t>(sizeof(float)); }

// dgamma / dbeta (float32, length D) may be null; workspace as sized by cueq_layer_norm_bwd_workspace.
extern "C" int cueq_layer_norm_bwd(int32_t dtype, int64_t rows, int64_t D, const void* dy, const void* x, const float* mean, const float* rstd,
                                   const void* gamma, void* dx, float* dgamma, float* dbeta, void* workspace, int64_t workspace_bytes,
                                   void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(is_io(dtype), CUEQ_ERR_UNSUPPORTED, "layer_norm: dtype must be float32 or bfloat16");
  CUEQ_REQUIRE(D > 0 && D <= 64 * kLnMaxPerLane, CUEQ_ERR_UNSUPPORTED, "layer_norm: hidden size must be in [1, %d]", 64 * kLnMaxPerLane);
  const int64_t nb = ln_bwd_blocks(rows);
  if (rows <= 0) {
    if (dgamma) CUEQ_CHECK_HIP(hipMemsetAsync(dgamma, 0, D * sizeof(float), stream));
    if (dbeta) CUEQ_CHECK_HIP(hipMemsetAsync(dbeta, 0, D * sizeof(float), stream));
    return CUEQ_OK;
  }
  CUEQ_REQUIRE(dy && x && mean && rstd && dx, CUEQ_ERR_INVALID, "layer_norm: null operand");
  CUEQ_REQUIRE(workspace && workspace_bytes >= cueq_layer_norm_bwd_workspace(rows, D), CUEQ_ERR_INVALID, "layer_norm: workspace too small");
  float* part = static_cast<float*>(workspace);
  const int rpb = static_cast<int>((rows + nb - 1) / nb);
  const size_t sh = 4 * 2 * D * sizeof(float);
  {
    KernelTimer timer("layer_norm_bwd", stream);
    const bool al16 = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(dy) | reinterpret_cast<uintptr_t>(dx) | reinterpret_cast<uintptr_t>(gamma)) & 15) == 0;
    const int nq = static_cast<int>((D + 63) / 64);
    if (al16 && (D == 32 || D == 64 || D == 128 || D == 256 || D == 512)) {
      const int L = static_cast<int>(D / 8);
#define LNB8(T, LL) hipLaunchKernelGGL((ln_bwd_rows8<T, LL>), dim3(static_cast<unsigned>(nb)), dim3(256), sh, stream, static_cast<const T*>(dy), static_cast<const T*>(x), mean, rstd, static_cast<const T*>(gamma), static_cast<T*>(dx), part, rows, rpb)
#define LNB8_L(T) do { switch (L) { case 4: LNB8(T, 4); break; case 8: LNB8(T, 8); break; case 16: LNB8(T, 16); break; case 32: LNB8(T, 32); break; default: LNB8(T, 64); } } while (0)
      TRI_DISPATCH(dtype, LNB8_L(float), LNB8_L(uint16_t), LNB8_L(f16bits));
#undef LNB8_L
#undef LNB8
    } else {
#define LN_BWD(T, NQ) hipLaunchKernelGGL((ln_bwd_kernel<T, NQ>), dim3(static_cast<unsigned>(nb)), dim3(256), sh, stream, static_cast<const T*>(dy), static_cast<const T*>(x), mean, rstd, static_cast<const T*>(gamma), static_cast<T*>(dx), part, rows, static_cast<int>(D), rpb)
#define LN_BWD_NQ(T) do { if (nq <= 1) LN_BWD(T, 1); else if (nq <= 2) LN_BWD(T, 2); else if (nq <= 4) LN_BWD(T, 4); else if (nq <= 8) LN_BWD(T, 8); else LN_BWD(T, 16); } while (0)
    TRI_DISPATCH(dtype, LN_BWD_NQ(float), LN_BWD_NQ(uint16_t), LN_BWD_NQ(f16bits));
#undef LN_BWD_NQ
#undef LN_BWD
    }
  }
  CUEQ_CHECK_HIP(hipGetLastError());
  const unsigned g = static_cast<unsigned>((D + 255) / 256);
  if (dgamma) hipLaunchKernelGGL(fold_partials_kernel<float>, dim3(g), dim3(256), 0, stream, part, dgamma, nb, D, 0);
  CUEQ_CHECK_HIP(hipGetLastError());
  if (dbeta) hipLaunchKernelGGL(fold_partials_kernel<float>, dim3(g), dim3(256), 0, stream, part + nb * D, dbeta, nb, D, 0);
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

static bool ln_t_ok(int32_t dtype, int64_t M, int64_t D, const void* a, const void* b, const void* c) {
  const int epv = dtype == CUEQ_F32 ? 4 : 8;
  return D > 0 && D <= kLnTMaxD && D % epv == 0 && M % epv == 0 &&
         ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c)) & 15) == 0;
}

extern "C" int cueq_layer_norm_t_fwd(int32_t dtype, int64_t M, int64_t D, const void* x_t, const void* gamma, const void* beta, double eps,
                                     void* y, float* mean, float* rstd, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(is_io(dtype), CUEQ_ERR_UNSUPPORTED, "layer_norm_t: dtype must be float32 or bfloat16");
  if (M <= 0) return CUEQ_OK;
  CUEQ_REQUIRE(x_t && y && mean && rstd, CUEQ_ERR_INVALID, "layer_norm_t: null operand");
  CUEQ_REQUIRE(ln_t_ok(dtype, M, D, x_t, y, nullptr), CUEQ_ERR_UNSUPPORTED,
               "layer_norm_t: D must be at most %d, D and M multiples of 16 bytes of elements, pointers 16-byte aligned", kLnTMaxD);
  const int64_t mt = dtype == CUEQ_F32 ? 32 : 64;
  const int64_t ntiles = (M + mt - 1) / mt;
  CUEQ_REQUIRE(ntiles < (1ll << 31), CUEQ_ERR_TOO_LARGE, "layer_norm_t: too many rows");
  const size_t fwd_lds = static_cast<size_t>(D) * 132;
  KernelTimer timer("layer_norm_t_fwd", stream);
  const bool half = dtype == CUEQ_F16;
  if (dtype != CUEQ_F32 && (D == 64 || D == 128) && D * M + 256 < (1ll << 32) &&
      ((reinterpret_cast<uintptr_t>(mean) | reinterpret_cast<uintptr_t>(rstd)) & 7) == 0) {
    // one lane per column pair and half of d, 64 columns per wavefront, four wavefronts per block, two blocks per CU
    int64_t nb = (ntiles + 3) / 4;
    if (nb > 2 * device_cus()) nb = 2 * device_cus();
    const size_t lds = static_cast<size_t>(4 * 64) * (2 * D + 16);
#define LNTC_F(FT, DD)                                                                                                                             \
  do {                                                                                                                                       \
    auto kfn = ln_t_fwd_cols_kernel<FT, DD>;                                                                                                     \
    CUEQ_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kfn), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds))); \
    hipLaunchKernelGGL(kfn, dim3(static_cast<unsigned>(nb)), dim3(256), lds, stream, static_cast<const FT*>(x_t),                       \
                       static_cast<const FT*>(gamma), static_cast<const FT*>(beta), static_cast<FT*>(y), mean, rstd, M,    \
                       static_cast<float>(eps));                                                                                             \
  } while (0)
#define LNTC(DD) do { if (half) LNTC_F(f16bits, DD); else LNTC_F(uint16_t, DD); } while (0)
    if (D == 64) LNTC(64); else LNTC(128);
#undef LNTC
#undef LNTC_F
    CUEQ_CHECK_HIP(hipGetLastError());
    return CUEQ_OK;
  }
  TRI_DISPATCH(dtype,
               hipLaunchKernelGGL(ln_t_fwd_kernel<float>, dim3(static_cast<unsigned>(ntiles)), dim3(256), fwd_lds, stream, static_cast<const float*>(x_t), static_cast<const float*>(gamma), static_cast<const float*>(beta), static_cast<float*>(y), mean, rstd, M, static_cast<int>(D), static_cast<float>(eps)),
               hipLaunchKernelGGL(ln_t_fwd_kernel<uint16_t>, dim3(static_cast<unsigned>(ntiles)), dim3(256), fwd_lds, stream, static_cast<const uint16_t*>(x_t), static_cast<const uint16_t*>(gamma), static_cast<const uint16_t*>(beta), static_cast<uint16_t*>(y), mean, rstd, M, static_cast<int>(D), static_cast<float>(eps)),
               hipLaunchKernelGGL(ln_t_fwd_kernel<f16bits>, dim3(static_cast<unsigned>(ntiles)), dim3(256), fwd_lds, stream, static_cast<const f16bits*>(x_t), static_cast<const f16bits*>(gamma), static_cast<const f16bits*>(beta), static_cast<f16bits*>(y), mean, rstd, M, static_cast<int>(D), static_cast<float>(eps)));
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

static int64_t ln_t_bwd_blocks(int32_t dtype, int64_t M) {
  const int64_t mt = dtype == CUEQ_F32 ? 32 : 64;
  const int64_t ntiles = (M + mt - 1) / mt;
  const int64_t nb = static_cast<int64_t>(device_cus()) * 8;
  return ntiles < nb ? (ntiles < 1 ? 1 : ntiles) : nb;
}

extern "C" int64_t cueq_layer_norm_t_bwd_workspace(int32_t dtype, int64_t M, int64_t D) {
  return ln_t_bwd_blocks(dtype, M) * 2 * D * static_cast<int64_t>(sizeof(float));
}

extern "C" int cueq_layer_norm_t_bwd(int32_t dtype, int64_t M, int64_t D, const void* dy, const void* x_t, const float* mean, const float* rstd,
                                     const void* gamma, void* dx_t, float* dgamma, float* dbeta, void* workspace, int64_t workspace_bytes,
                                     void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(is_io(dtype), CUEQ_ERR_UNSUPPORTED, "layer_norm_t: dtype must be float32 or bfloat16");
  if (M <= 0) {
    if (dgamma) CUEQ_CHECK_HIP(hipMemsetAsync(dgamma, 0, D * sizeof(float), stream));
    if (dbeta) CUEQ_CHECK_HIP(hipMemsetAsync(dbeta, 0, D * sizeof(float), stream));
    return CUEQ_OK;
  }
  CUEQ_REQUIRE(dy && x_t && mean && rstd && dx_t, CUEQ_ERR_INVALID, "layer_norm_t: null operand");
  CUEQ_REQUIRE(ln_t_ok(dtype, M, D, x_t, dy, dx_t), CUEQ_ERR_UNSUPPORTED,
               "layer_norm_t: D must be at most %d, D and M multiples of 16 bytes of elements, pointers 16-byte aligned", kLnTMaxD);
  const int need_affine = (dgamma || dbeta) ? 1 : 0;
  CUEQ_REQUIRE(!need_affine || (workspace && workspace_bytes >= cueq_layer_norm_t_bwd_workspace(dtype, M, D)), CUEQ_ERR_INVALID,
               "layer_norm_t: workspace too small");
  const int64_t mt = dtype == CUEQ_F32 ? 32 : 64;
  const int64_t ntiles = (M + mt - 1) / mt;
  const int64_t nb = ln_t_bwd_blocks(dtype, M);
  float* part = static_cast<float*>(workspace);
  const int64_t es = dtype == CUEQ_F32 ? 4 : 2;
  const bool half = dtype == CUEQ_F16;
  if (dtype != CUEQ_F32 && !need_affine && (D == 64 || D == 128) && D * M + 256 < (1ll << 32) &&
      ((reinterpret_cast<uintptr_t>(mean) | reinterpret_cast<uintptr_t>(rstd)) & 7) == 0) {
    // one lane per column pair and half of d, 64 columns per wavefront, four wavefronts per block, two blocks per CU
    int64_t nbc = (ntiles + 3) / 4;
    if (nbc > 2 * device_cus()) nbc = 2 * device_cus();
    const size_t lds = static_cast<size_t>(4 * 64) * (2 * D + 16);
    KernelTimer timer("layer_norm_t_bwd", stream);
#define LNTC_F(FT, DD)                                                                                                                             \
  do {                                                                                                                                       \
    auto kfn = ln_t_bwd_cols_kernel<FT, DD>;                                                                                                     \
    CUEQ_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kfn), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds))); \
    hipLaunchKernelGGL(kfn, dim3(static_cast<unsigned>(nbc)), dim3(256), lds, stream, static_cast<const FT*>(dy),                       \
                       static_cast<const FT*>(x_t), mean, rstd, static_cast<const FT*>(gamma), static_cast<FT*>(dx_t), M); \
  } while (0)
#define LNTC(DD) do { if (half) LNTC_F(f16bits, DD); else LNTC_F(uint16_t, DD); } while (0)
    if (D == 64) LNTC(64); else LNTC(128);
#undef LNTC
#undef LNTC_F
    CUEQ_CHECK_HIP(hipGetLastError());
    return CUEQ_OK;
  }
  const size_t bwd_lds = static_cast<size_t>(((D * 132 + 15) & ~15ll) + mt * (D * es + 4));
  {
    KernelTimer timer("layer_norm_t_bwd", stream);
    TRI_DISPATCH(dtype,
                 hipLaunchKernelGGL(ln_t_bwd_kernel<float>, dim3(static_cast<unsigned>(nb)), dim3(256), bwd_lds, stream, static_cast<const float*>(dy), static_cast<const float*>(x_t), mean, rstd, static_cast<const float*>(gamma), static_cast<float*>(dx_t), part, M, static_cast<int>(D), ntiles, need_affine),
                 hipLaunchKernelGGL(ln_t_bwd_kernel<uint16_t>, dim3(static_cast<unsigned>(nb)), dim3(256), bwd_lds, stream, static_cast<const uint16_t*>(dy), static_cast<const uint16_t*>(x_t), mean, rstd, static_cast<const uint16_t*>(gamma), static_cast<uint16_t*>(dx_t), part, M, static_cast<int>(D), ntiles, need_affine),
                 hipLaunchKernelGGL(ln_t_bwd_kernel<f16bits>, dim3(static_cast<unsigned>(nb)), dim3(256), bwd_lds, stream, static_cast<const f16bits*>(dy), static_cast<const f16bits*>(x_t), mean, rstd, static_cast<const f16bits*>(gamma), static_cast<f16bits*>(dx_t), part, M, static_cast<int>(D), ntiles, need_affine));
  }
  CUEQ_CHECK_HIP(hipGetLastError());
  const unsigned g = static_cast<unsigned>((D + 255) / 256);
  if (dgamma) hipLaunchKernelGGL(fold_partials_kernel<float>, dim3(g), dim3(256), 0, stream, part, dgamma, nb, D, 0);
  CUEQ_CHECK_HIP(hipGetLastError());
  if (dbeta) hipLaunchKernelGGL(fold_partials_kernel<float>, dim3(g), dim3(256), 0, stream, part + nb * D, dbeta, nb, D, 0);
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

extern "C" int cueq_gate_fwd(int32_t dtype, int64_t rows, int64_t cols, const float* u, const float* v, const void* bias_u, const void* bias_v,
                             int32_t bias_axis, const void* mask, int32_t mask_axis, void* out, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(is_io(dtype), CUEQ_ERR_UNSUPPORTED, "gate: dtype must be float32 or bfloat16");
  const int64_t n = rows * cols;
  if (n <= 0) return CUEQ_OK;
  CUEQ_REQUIRE(u && v && out, CUEQ_ERR_INVALID, "gate: null operand");
  CUEQ_REQUIRE((n + 255) / 256 < (1ll << 31), CUEQ_ERR_TOO_LARGE, "gate: too many elements");
  const dim3 grid(static_cast<unsigned>((n + 255) / 256));
  KernelTimer timer("gate_fwd", stream);
  TRI_DISPATCH(dtype,
               hipLaunchKernelGGL(gate_fwd_kernel<float>, grid, dim3(256), 0, stream, u, v, static_cast<const float*>(bias_u), static_cast<const float*>(bias_v), bias_axis, static_cast<const float*>(mask), mask_axis, static_cast<float*>(out), rows, cols),
               hipLaunchKernelGGL(gate_fwd_kernel<uint16_t>, grid, dim3(256), 0, stream, u, v, static_cast<const uint16_t*>(bias_u), static_cast<const uint16_t*>(bias_v), bias_axis, static_cast<const uint16_t*>(mask), mask_axis, static_cast<uint16_t*>(out), rows, cols),
               hipLaunchKernelGGL(gate_fwd_kernel<f16bits>, grid, dim3(256), 0, stream, u, v, static_cast<const f16bits*>(bias_u), static_cast<const f16bits*>(bias_v), bias_axis, static_cast<const f16bits*>(mask), mask_axis, static_cast<f16bits*>(out), rows, cols));
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

extern "C" int cueq_gate_bwd(int32_t dtype, int64_t rows, int64_t cols, const void* dout, const float* u, const float* v, const void* bias_u,
                             const void* bias_v, int32_t bias_axis, const void* mask, int32_t mask_axis, void* du, void* dv, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(is_io(dtype), CUEQ_ERR_UNSUPPORTED, "gate: dtype must be float32 or bfloat16");
  const int64_t n = rows * cols;
  if (n <= 0) return CUEQ_OK;
  CUEQ_REQUIRE(dout && u && v && du && dv, CUEQ_ERR_INVALID, "gate: null operand");
  CUEQ_REQUIRE((n + 255) / 256 < (1ll << 31), CUEQ_ERR_TOO_LARGE, "gate: too many elements");
  const dim3 grid(static_cast<unsigned>((n + 255) / 256));
  KernelTimer timer("gate_bwd", stream);
  TRI_DISPATCH(dtype,
               hipLaunchKernelGGL(gate_bwd_kernel<float>, grid, dim3(256), 0, stream, static_cast<const float*>(dout), u, v, static_cast<const float*>(bias_u), static_cast<const float*>(bias_v), bias_axis, static_cast<const float*>(mask), mask_axis, static_cast<float*>(du), static_cast<float*>(dv), rows, cols),
               hipLaunchKernelGGL(gate_bwd_kernel<uint16_t>, grid, dim3(256), 0, stream, static_cast<const uint16_t*>(dout), u, v, static_cast<const uint16_t*>(bias_u), static_cast<const uint16_t*>(bias_v), bias_axis, static_cast<const uint16_t*>(mask), mask_axis, static_cast<uint16_t*>(du), static_cast<uint16_t*>(dv), rows, cols),
               hipLaunchKernelGGL(gate_bwd_kernel<f16bits>, grid, dim3(256), 0, stream, static_cast<const f16bits*>(dout), u, v, static_cast<const f16bits*>(bias_u), static_cast<const f16bits*>(bias_v), bias_axis, static_cast<const f16bits*>(mask), mask_axis, static_cast<f16bits*>(du), static_cast<f16bits*>(dv), rows, cols));
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

// out[r] = sum_c in[r][c]   (float32 result)
extern "C" int cueq_sum_cols(int32_t dtype, int64_t rows, int64_t cols, const void* in, float* out, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(is_io(dtype), CUEQ_ERR_UNSUPPORTED, "sum_cols: dtype must be float32 or bfloat16");
  if (rows <= 0) return CUEQ_OK;
  CUEQ_REQUIRE(in && out, CUEQ_ERR_INVALID, "sum_cols: null operand");
  const dim3 grid(static_cast<unsigned>((rows + 3) / 4));
  TRI_DISPATCH(dtype,
               hipLaunchKernelGGL(sum_cols_kernel<float>, grid, dim3(256), 0, stream, static_cast<const float*>(in), out, rows, cols),
               hipLaunchKernelGGL(sum_cols_kernel<uint16_t>, grid, dim3(256), 0, stream, static_cast<const uint16_t*>(in), out, rows, cols),
               hipLaunchKernelGGL(sum_cols_kernel<f16bits>, grid, dim3(256), 0, stream, static_cast<const f16bits*>(in), out, rows, cols));
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

// row blocks of the first stage: enough of them that the launch fills the chip (about 2048 workgroups with the column
// blocks), at least 8 rows each, at most 1024
static int64_t sum_rows_blocks(int64_t rows, int64_t cols) {
  const int64_t col_blocks = (cols + 255) / 256;
  int64_t nb = (2048 + col_blocks - 1) / col_blocks;
  if (nb > (rows + 7) / 8) nb = (rows + 7) / 8;
  if (nb > 1024) nb = 1024;
  return nb < 1 ? 1 : nb;
}

extern "C" int64_t cueq_sum_rows_workspace(int64_t rows, int64_t cols) { return sum_rows_blocks(rows, cols) * cols * static_cast<int64_t>(sizeof(float)); }

// out[c] = sum_r in[r][c]   (float32 result, deterministic two-stage reduction)
extern "C" int cueq_sum_rows(int32_t dtype, int64_t rows, int64_t cols, const void* in, float* out, void* workspace, int64_t workspace_bytes,
                             void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(is_io(dtype), CUEQ_ERR_UNSUPPORTED, "sum_rows: dtype must be float32 or bfloat16");
  if (cols <= 0) return CUEQ_OK;
  CUEQ_REQUIRE(out, CUEQ_ERR_INVALID, "sum_rows: null output");
  if (rows <= 0) {
    CUEQ_CHECK_HIP(hipMemsetAsync(out, 0, cols * sizeof(float), stream));
    return CUEQ_OK;
  }
  CUEQ_REQUIRE(in && workspace && workspace_bytes >= cueq_sum_rows_workspace(rows, cols), CUEQ_ERR_INVALID, "sum_rows: workspace too small");
  if (rows <= 4096 && (cols + 63) / 64 >= 128) {  // few rows, enough column blocks to fill the chip: one launch
    const dim3 grid1(static_cast<unsigned>((cols + 63) / 64));
    TRI_DISPATCH(dtype,
                 hipLaunchKernelGGL(sum_rows_lds_kernel<float>, grid1, dim3(1024), 0, stream, static_cast<const float*>(in), out, rows, cols),
                 hipLaunchKernelGGL(sum_rows_lds_kernel<uint16_t>, grid1, dim3(1024), 0, stream, static_cast<const uint16_t*>(in), out, rows, cols),
                 hipLaunchKernelGGL(sum_rows_lds_kernel<f16bits>, grid1, dim3(1024), 0, stream, static_cast<const f16bits*>(in), out, rows, cols));
    CUEQ_CHECK_HIP(hipGetLastError());
    return CUEQ_OK;
  }
  const int64_t nb = sum_rows_blocks(rows, cols);
  const int64_t rpb = (rows + nb - 1) / nb;
  float* part = static_cast<float*>(workspace);
  const dim3 grid(static_cast<unsigned>((cols + 255) / 256), static_cast<unsigned>(nb));
  TRI_DISPATCH(dtype,
               hipLaunchKernelGGL(sum_rows_partial_kernel<float>, grid, dim3(256), 0, stream, static_cast<const float*>(in), part, rows, cols, rpb),
               hipLaunchKernelGGL(sum_rows_partial_kernel<uint16_t>, grid, dim3(256), 0, stream, static_cast<const uint16_t*>(in), part, rows, cols, rpb),
               hipLaunchKernelGGL(sum_rows_partial_kernel<f16bits>, grid, dim3(256), 0, stream, static_cast<const f16bits*>(in), part, rows, cols, rpb));
  CUEQ_CHECK_HIP(hipGetLastError());
  hipLaunchKernelGGL(fold_partials_kernel<float>, dim3(static_cast<unsigned>((cols + 255) / 256)), dim3(256), 0, stream, part, out, nb, cols, 0);
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}
