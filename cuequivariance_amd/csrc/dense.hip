// Dense segmented contractions on the matrix cores (MFMA), for equivariant Linear and
// fully-connected tensor products with shared weights.
//
// After the Clebsch-Gordan modes are flattened, every path of such a polynomial is a small GEMM
//     C[z, c_seg, :] (+)= alpha * s[z] * A[z, a_seg, :] @ W_p            (K x N weight block W_p)
// with an optional per-row scalar s[z] (the second operand of a fully-connected product, whose
// multiplicity is 1).  Stands for the closed modules the reference calls at
// cuequivariance_torch/cuequivariance_torch/primitives/segmented_polynomial_fused_tp.py:27-72
// (FusedTensorProductOp3 / Op4).
//
// seg_gemm: one workgroup per (weight block, persistent slot).  Each wavefront owns 32 output
// columns and keeps its K x 32 slice of the weight block in registers for the whole kernel; row
// tiles of A (32 rows x K) stream through LDS (double buffered, 16-byte coalesced global loads).
// The contraction index is permuted so that each lane reads contiguous LDS words.
// seg_outer: weight gradient, contraction over the batch; both MFMA operands are read straight
// from global memory (the batch index is the MFMA k index), per-workgroup partial sums are folded
// in a fixed order: no atomics.

#include <vector>

#include "common.h"
#include "cw_common.h"
#include "u1d_spec.h"

namespace cueq {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

struct GemmProblem {
  int64_t a_off, c_off, b_off;
  double alpha;
  int32_t s_col, trans_b;
  int32_t accumulate, pad;
};

constexpr int kMaxProblems = 65535;  // grid.y

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(uint16_t v) { return bf16_bits_to_float(v); }
__device__ __forceinline__ void from_float(float& d, float v) { d = v; }
__device__ __forceinline__ void from_float(uint16_t& d, float v) { d = float_to_bf16_bits(v); }
__device__ __forceinline__ double to_float(double v) { return v; }
__device__ __forceinline__ void from_float(double& d, double v) { d = v; }
__device__ __forceinline__ void from_float(float& d, double v) { d = static_cast<float>(v); }

// ------------------------------------------------------------------------------------------------
// fp32: v_mfma_f32_32x32x2_f32.  A operand lane l holds A[l%32][k(l/32, step)], B operand B[k][l%32].
// A row tile is RT x 32 rows; one barrier per tile.
// ------------------------------------------------------------------------------------------------
template <int K, int NW, int RT>
__global__ void __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(2))) seg_gemm_f32(
    const float* __restrict__ A, int64_t lda, const float* __restrict__ B, const float* __restrict__ S, int64_t lds_,
    float* __restrict__ C, int64_t ldc, int64_t rows, int N, const GemmProblem* __restrict__ probs) {
  constexpr int KH = K / 2;        // contraction indices handled by one lane half
  constexpr int LDA = K + 4;       // padded LDS row (floats)
  constexpr int TM = 32 * RT;      // rows per tile
  extern __shared__ float smem[];  // 2 x TM x LDA
  const GemmProblem pr = probs[blockIdx.y];
  constexpr int nthreads = 64 * NW;
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, c = lane & 31, h = lane >> 5;
  const int n0 = wave * 32;

  float breg[KH];
#pragma unroll
  for (int s = 0; s < KH; ++s) {
    const int k = h * KH + s;
    breg[s] = pr.trans_b ? B[pr.b_off + static_cast<int64_t>(n0 + c) * K + k] : B[pr.b_off + static_cast<int64_t>(k) * N + n0 + c];
  }

  const int64_t ntiles = (rows + TM - 1) / TM;
  constexpr int V4_PER_ROW = K / 4;
  constexpr int total_v4 = TM * V4_PER_ROW;
  constexpr int per_thread = (total_v4 + nthreads - 1) / nthreads;
  float4 stage[per_thread];

  auto load_tile = [&](int64_t t) {
#pragma unroll
    for (int q = 0; q < per_thread; ++q) {
      const int e = tid + q * nthreads;
      if (e < total_v4) {
        const int r = e / V4_PER_ROW, v = e - r * V4_PER_ROW;
        int64_t row = t * TM + r;
        if (row >= rows) row = rows - 1;
        stage[q] = *reinterpret_cast<const float4*>(A + row * lda + pr.a_off + v * 4);
      }
    }
  };
  auto store_tile = [&](int buf) {
    float* dst = smem + buf * TM * LDA;
#pragma unroll
    for (int q = 0; q < per_thread; ++q) {
      const int e = tid + q * nthreads;
      if (e < total_v4) {
        const int r = e / V4_PER_ROW, v = e - r * V4_PER_ROW;
        *reinterpret_cast<float4*>(dst + r * LDA + v * 4) = stage[q];
      }
    }
  };

  const float alpha = static_cast<float>(pr.alpha);
  int64_t t = blockIdx.x;
  if (t < ntiles) load_tile(t);
  int buf = 0;
  for (; t < ntiles; t += gridDim.x) {
    store_tile(buf);
    __syncthreads();
    const int64_t tn = t + gridDim.x;
    if (tn < ntiles) load_tile(tn);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const float* a = smem + (buf * TM + rt * 32 + c) * LDA + h * KH;
      // all LDS reads of the sub-tile are issued before the first MFMA; they return in order
      float4 av[KH / 4];
#pragma unroll
      for (int q = 0; q < KH / 4; ++q) av[q] = *reinterpret_cast<const float4*>(a + 4 * q);
      floatx16 acc = {0};
#pragma unroll
      for (int q = 0; q < KH / 4; ++q) {
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[q].x, breg[4 * q + 0], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[q].y, breg[4 * q + 1], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[q].z, breg[4 * q + 2], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[q].w, breg[4 * q + 3], acc, 0, 0, 0);
      }
      // epilogue: uniform sub-tile base + 32-bit lane offset
      const int64_t r0 = t * TM + rt * 32;
      float* __restrict__ ctile = C + r0 * ldc + pr.c_off + n0;
      const float* __restrict__ stile = S + r0 * lds_ + (pr.s_col >= 0 ? pr.s_col : 0);
      const int64_t rows_left = rows - r0;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int r = 8 * (v >> 2) + 4 * h + (v & 3);
        if (r < rows_left) {
          float val = alpha * acc[v];
          if (pr.s_col >= 0) val *= stile[r * static_cast<int>(lds_)];
          const int off = r * static_cast<int>(ldc) + c;
          if (pr.accumulate) val += ctile[off];
          ctile[off] = val;
        }
      }
    }
    buf ^= 1;
  }
}

// ------------------------------------------------------------------------------------------------
// bf16 in / bf16 out, fp32 accumulate: v_mfma_f32_32x32x16_bf16 (lane half h supplies 8 of the 16 k)
// ------------------------------------------------------------------------------------------------
template <int K, int NW>
__global__ void __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(4))) seg_gemm_bf16(const uint16_t* __restrict__ A, int64_t lda,
                                                     const uint16_t* __restrict__ B, const uint16_t* __restrict__ S,
                                                     int64_t lds_, uint16_t* __restrict__ C, int64_t ldc, int64_t rows,
                                                     int N, const GemmProblem* __restrict__ probs) {
  constexpr int KH = K / 2;
  constexpr int STEPS = K / 16;
  constexpr int LDA = K + 8;  // padded LDS row (bf16)
  extern __shared__ float smem[];
  uint16_t* sm = reinterpret_cast<uint16_t*>(smem);
  const GemmProblem pr = probs[blockIdx.y];
  constexpr int nthreads = 64 * NW;
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, c = lane & 31, h = lane >> 5;
  const int n0 = wave * 32;

  bf16x8 breg[STEPS];
#pragma unroll
  for (int q = 0; q < STEPS; ++q) {
    uint16_t tmp[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int k = h * KH + q * 8 + e;
      tmp[e] = pr.trans_b ? B[pr.b_off + static_cast<int64_t>(n0 + c) * K + k] : B[pr.b_off + static_cast<int64_t>(k) * N + n0 + c];
    }
    breg[q] = *reinterpret_cast<bf16x8*>(tmp);
  }

  const int64_t ntiles = (rows + 31) / 32;
  constexpr int V8_PER_ROW = K / 8;  // 16-byte chunks per row
  constexpr int total = 32 * V8_PER_ROW;
  constexpr int per_thread = (total + nthreads - 1) / nthreads;
  uint4 stage[per_thread];

  auto load_tile = [&](int64_t t) {
#pragma unroll
    for (int q = 0; q < per_thread; ++q) {
      const int e = tid + q * nthreads;
      if (e < total) {
        const int r = e / V8_PER_ROW, v = e - r * V8_PER_ROW;
        int64_t row = t * 32 + r;
        if (row >= rows) row = rows - 1;
        stage[q] = *reinterpret_cast<const uint4*>(A + row * lda + pr.a_off + v * 8);
      }
    }
  };
  auto store_tile = [&](int buf) {
    uint16_t* dst = sm + buf * 32 * LDA;
#pragma unroll
    for (int q = 0; q < per_thread; ++q) {
      const int e = tid + q * nthreads;
      if (e < total) {
        const int r = e / V8_PER_ROW, v = e - r * V8_PER_ROW;
        *reinterpret_cast<uint4*>(dst + r * LDA + v * 8) = stage[q];
      }
    }
  };

  int64_t t = blockIdx.x;
  if (t < ntiles) load_tile(t);
  int buf = 0;
  for (; t < ntiles; t += gridDim.x) {
    store_tile(buf);
    __syncthreads();
    const int64_t tn = t + gridDim.x;
    if (tn < ntiles) load_tile(tn);
    const uint16_t* a = sm + buf * 32 * LDA + c * LDA + h * KH;
    floatx16 acc = {0};
#pragma unroll
    for (int q = 0; q < STEPS; ++q) {
      const bf16x8 av = *reinterpret_cast<const bf16x8*>(a + q * 8);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, breg[q], acc, 0, 0, 0);
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int64_t row = t * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
      if (row < rows) {
        float val = static_cast<float>(pr.alpha) * acc[v];
        if (pr.s_col >= 0) val *= bf16_bits_to_float(S[row * lds_ + pr.s_col]);
        uint16_t* dst = C + row * ldc + pr.c_off + n0 + c;
        if (pr.accumulate) val += bf16_bits_to_float(*dst);
        *dst = float_to_bf16_bits(val);
      }
    }
    buf ^= 1;
  }
}

// ------------------------------------------------------------------------------------------------
// generic fallback (any K, N; float, double, bf16): one thread per output element
// ------------------------------------------------------------------------------------------------
template <typename IO, typename ACC>
__global__ void __launch_bounds__(256) seg_gemm_simple(const IO* __restrict__ A, int64_t lda, const IO* __restrict__ B,
                                                       const IO* __restrict__ S, int64_t lds_, IO* __restrict__ C,
                                                       int64_t ldc, int64_t rows, int K, int N, const GemmProblem* __restrict__ probs) {
  const GemmProblem pr = probs[blockIdx.y];
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tid >= rows * N) return;
  const int64_t row = tid / N;
  const int n = static_cast<int>(tid - row * N);
  ACC acc = 0;
  for (int k = 0; k < K; ++k) {
    const ACC b = pr.trans_b ? static_cast<ACC>(to_float(B[pr.b_off + static_cast<int64_t>(n) * K + k]))
                             : static_cast<ACC>(to_float(B[pr.b_off + static_cast<int64_t>(k) * N + n]));
    acc += static_cast<ACC>(to_float(A[row * lda + pr.a_off + k])) * b;
  }
  acc *= static_cast<ACC>(pr.alpha);
  if (pr.s_col >= 0) acc *= static_cast<ACC>(to_float(S[row * lds_ + pr.s_col]));
  IO* dst = C + row * ldc + pr.c_off + n;
  if (pr.accumulate) acc += static_cast<ACC>(to_float(*dst));
  from_float(*dst, acc);
}

// ------------------------------------------------------------------------------------------------
// weight gradient: dW[k][n] = sum over entries e and rows z of alpha_e * s_e[z] * A[z, a_off_e + k] * G[z, c_off_e + n]
// partial[slot][k][n] per workgroup, folded afterwards.
// ------------------------------------------------------------------------------------------------
struct OuterEntry {
  int64_t a_off, c_off;
  double alpha;
  int32_t s_col, pad;
};
struct OuterProblem {
  const OuterEntry* e;  // device pointer
  int32_t n_entries;
  int32_t trans_out;  // 0: dW[k][n], 1: dW[n][k]
};

template <typename IO, int NB>
__global__ void __launch_bounds__(512) seg_outer_mfma(const IO* __restrict__ A, int64_t lda, const IO* __restrict__ G,
                                                      int64_t ldg, const IO* __restrict__ S, int64_t lds_,
                                                      float* __restrict__ partial, int64_t rows, int K,
                                                      int64_t rows_per_block, OuterProblem pr) {
  // wavefront w owns k-block w (32 rows of dW) and all NB column blocks; the batch index is the MFMA k
  // index: lane half h feeds row zi + 2q + h.  Eight row pairs are loaded before their MFMAs are issued.
  constexpr int N = NB * 32;
  constexpr int UNROLL = 8;
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, c = lane & 31, h = lane >> 5;
  const int k0 = wave * 32;
  floatx16 acc[NB];
#pragma unroll
  for (int j = 0; j < NB; ++j) acc[j] = floatx16{0};
  const int64_t z_begin = static_cast<int64_t>(blockIdx.x) * rows_per_block;
  const int64_t z_end = z_begin + rows_per_block < rows ? z_begin + rows_per_block : rows;
  for (int ent = 0; ent < pr.n_entries; ++ent) {
    const OuterEntry en = pr.e[ent];
    const float alpha = static_cast<float>(en.alpha);
    for (int64_t zi = z_begin; zi < z_end; zi += 2 * UNROLL) {
      float a[UNROLL], g[UNROLL][NB];
#pragma unroll
      for (int q = 0; q < UNROLL; ++q) {
        const int64_t z = zi + 2 * q + h;
        const bool ok = z < z_end;
        const int64_t zz = ok ? z : z_end - 1;
        float av = to_float(A[zz * lda + en.a_off + k0 + c]) * alpha;
        if (en.s_col >= 0) av *= to_float(S[zz * lds_ + en.s_col]);
        a[q] = ok ? av : 0.f;
#pragma unroll
        for (int j = 0; j < NB; ++j) g[q][j] = to_float(G[zz * ldg + en.c_off + j * 32 + c]);
      }
#pragma unroll
      for (int q = 0; q < UNROLL; ++q)
#pragma unroll
        for (int j = 0; j < NB; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[q], g[q][j], acc[j], 0, 0, 0);
    }
  }
  float* out = partial + static_cast<int64_t>(blockIdx.x) * K * N;
#pragma unroll
  for (int j = 0; j < NB; ++j) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int k = k0 + 8 * (v >> 2) + 4 * h + (v & 3);
      const int n = j * 32 + c;
      out[pr.trans_out ? static_cast<int64_t>(n) * K + k : static_cast<int64_t>(k) * N + n] = acc[j][v];
    }
  }
}

template <typename IO, typename ACC>
__global__ void __launch_bounds__(256) seg_outer_simple(const IO* __restrict__ A, int64_t lda, const IO* __restrict__ G,
                                                        int64_t ldg, const IO* __restrict__ S, int64_t lds_,
                                                        ACC* __restrict__ partial, int64_t rows, int K, int N,
                                                        int64_t rows_per_block, OuterProblem pr) {
  const int64_t z_begin = static_cast<int64_t>(blockIdx.y) * rows_per_block;
  const int64_t z_end = z_begin + rows_per_block < rows ? z_begin + rows_per_block : rows;
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= K * N) return;
  const int k = e / N, n = e - k * N;
  ACC acc = 0;
  for (int ent = 0; ent < pr.n_entries; ++ent) {
    const OuterEntry en = pr.e[ent];
    for (int64_t z = z_begin; z < z_end; ++z) {
      ACC a = static_cast<ACC>(to_float(A[z * lda + en.a_off + k])) * static_cast<ACC>(en.alpha);
      if (en.s_col >= 0) a *= static_cast<ACC>(to_float(S[z * lds_ + en.s_col]));
      acc += a * static_cast<ACC>(to_float(G[z * ldg + en.c_off + n]));
    }
  }
  partial[static_cast<int64_t>(blockIdx.y) * K * N + (pr.trans_out ? static_cast<int64_t>(n) * K + k : static_cast<int64_t>(k) * N + n)] = acc;
}

// out[e] (+)= sum over slots (ascending) of partial[slot][e]
template <typename IO, typename ACC>
__global__ void __launch_bounds__(256) fold_slots(const ACC* __restrict__ partial, int nslots, int64_t n, IO* __restrict__ out,
                                                  int accumulate) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (e >= n) return;
  ACC acc = 0;
  for (int s = 0; s < nslots; ++s) acc += partial[static_cast<int64_t>(s) * n + e];
  if (accumulate) acc += static_cast<ACC>(to_float(out[e]));
  from_float(out[e], acc);
}

// row-wise dot: dS[z, s_col] (+)= alpha * sum_n G[z, c_off + n] * (A[z, a_off:a_off+K] @ W)[n]
template <typename IO, typename ACC>
__global__ void __launch_bounds__(256) seg_rowdot(const IO* __restrict__ A, int64_t lda, const IO* __restrict__ B,
                                                  const IO* __restrict__ G, int64_t ldg, IO* __restrict__ dS, int64_t lds_,
                                                  int64_t rows, int K, int N, GemmProblem pr) {
  // one wavefront per row: lanes over n, loop over k
  const int lane = threadIdx.x & 63;
  const int64_t row = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) >> 6;
  if (row >= rows) return;
  ACC acc = 0;
  for (int n = lane; n < N; n += 64) {
    ACC t = 0;
    for (int k = 0; k < K; ++k) {
      const ACC b = pr.trans_b ? static_cast<ACC>(to_float(B[pr.b_off + static_cast<int64_t>(n) * K + k]))
                               : static_cast<ACC>(to_float(B[pr.b_off + static_cast<int64_t>(k) * N + n]));
      t += static_cast<ACC>(to_float(A[row * lda + pr.a_off + k])) * b;
    }
    acc += t * static_cast<ACC>(to_float(G[row * ldg + pr.c_off + n]));
  }
  for (int d = 32; d >= 1; d >>= 1) acc += __shfl_xor(acc, d, 64);
  if (lane == 0) {
    acc *= static_cast<ACC>(pr.alpha);
    IO* dst = dS + row * lds_ + pr.s_col;
    if (pr.accumulate) acc += static_cast<ACC>(to_float(*dst));
    from_float(*dst, acc);
  }
}


// ------------------------------------------------------------------------------------------------
// Element-wise stages of the fully-connected product on the tiled GEMMs.  With T[:, t] = x1[:, i_seg] . W_p for every
// distinct (weight block, x1 segment) computed by cueq_gemm, every flattened path is
//   out[z, c_off + n] += coeff * x2[z, j] * T[z, t_off + n]
// (a "use" of T); the backward has the same shape with g in place of x1.  fc_combine sums the uses of every output
// block; fc_rowdot is the gradient of the multiplicity-one operand, dx2[z, j] += coeff * <x1[z, a_off : +K], G[z, g_off : +K]>.
// ------------------------------------------------------------------------------------------------
template <typename T> __device__ __forceinline__ constexpr int type_code() { return sizeof(T) == 4 ? CUEQ_F32 : CUEQ_BF16; }  // float / uint16_t (bf16 bits)
struct FcBlock { int32_t out_off, n, first_use, num_uses; };
struct FcUse { int32_t j, src_off; float coeff; int32_t pad; };

template <typename TS, typename TT, typename TO>
__global__ void __launch_bounds__(256) fc_combine_kernel(const TS* __restrict__ S, int64_t lds_, const TT* __restrict__ T, int64_t ldt,
                                                         TO* __restrict__ O, int64_t ldo, const FcBlock* __restrict__ blocks,
                                                         const FcUse* __restrict__ uses, int64_t Z, int max_n) {
  const FcBlock b = blocks[blockIdx.y];
  // a thread owns one column n of the block and walks rows; 256 threads cover 256 / max_n rows per pass
  const int rows_per_pass = 256 / max_n;
  const int n = threadIdx.x % max_n, r = threadIdx.x / max_n;
  if (n >= b.n || r >= rows_per_pass) return;
  for (int64_t z = static_cast<int64_t>(blockIdx.x) * rows_per_pass + r; z < Z; z += static_cast<int64_t>(gridDim.x) * rows_per_pass) {
    float acc = 0.f;
    for (int u = 0; u < b.num_uses; ++u) {
      const FcUse use = uses[b.first_use + u];
      acc = fmaf(use.coeff * load_as<float>(S, type_code<TS>(), z * lds_ + use.j), load_as<float>(T, type_code<TT>(), z * ldt + use.src_off + n), acc);
    }
    store_as<float>(O, type_code<TO>(), z * ldo + b.out_off + n, acc);
  }
}

// four adjacent columns per thread (16 / 8-byte accesses): blocks, offsets and row strides are multiples of four
__device__ __forceinline__ float4 fc_load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 fc_load4(const uint16_t* p) {
  const uint2 w = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xffff0000u), __uint_as_float(w.y << 16), __uint_as_float(w.y & 0xffff0000u));
}
__device__ __forceinline__ void fc_store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void fc_store4(uint16_t* p, float4 v) {
  uint16_t h[4];
  from_float(h[0], v.x); from_float(h[1], v.y); from_float(h[2], v.z); from_float(h[3], v.w);
  *reinterpret_cast<uint2*>(p) = make_uint2(static_cast<uint32_t>(h[0]) | (static_cast<uint32_t>(h[1]) << 16),
                                            static_cast<uint32_t>(h[2]) | (static_cast<uint32_t>(h[3]) << 16));
}

template <typename TS, typename TT, typename TO>
__global__ void __launch_bounds__(256) fc_combine_vec_kernel(const TS* __restrict__ S, int64_t lds_, const TT* __restrict__ T, int64_t ldt,
                                                             TO* __restrict__ O, int64_t ldo, const FcBlock* __restrict__ blocks,
                                                             const FcUse* __restrict__ uses, int64_t Z, int max_n) {
  const FcBlock b = blocks[blockIdx.y];
  const int tpr = max_n / 4;  // threads per row
  const int rows_per_pass = 256 / tpr;
  const int n = (threadIdx.x % tpr) * 4, r = threadIdx.x / tpr;
  if (n >= b.n || r >= rows_per_pass) return;
  for (int64_t z = static_cast<int64_t>(blockIdx.x) * rows_per_pass + r; z < Z; z += static_cast<int64_t>(gridDim.x) * rows_per_pass) {
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int u = 0; u < b.num_uses; ++u) {
      const FcUse use = uses[b.first_use + u];
      const float sc = use.coeff * load_as<float>(S, type_code<TS>(), z * lds_ + use.j);
      const float4 t = fc_load4(T + z * ldt + use.src_off + n);
      acc.x = fmaf(sc, t.x, acc.x); acc.y = fmaf(sc, t.y, acc.y); acc.z = fmaf(sc, t.z, acc.z); acc.w = fmaf(sc, t.w, acc.w);
    }
    fc_store4(O + z * ldo + b.out_off + n, acc);
  }
}

struct FcDotUse { int32_t j, a_off, g_off, k; float coeff; int32_t pad[3]; };

template <typename TX, typename TG>
__global__ void __launch_bounds__(256) fc_rowdot_kernel(const TX* __restrict__ X, int64_t ldx, const TG* __restrict__ G, int64_t ldg,
                                                        TX* __restrict__ D, int64_t ldd, int n2, const FcDotUse* __restrict__ uses,
                                                        int num_uses, int64_t Z) {
  // one wavefront per row; lane j keeps the running sum of column j (n2 <= 64)
  const int lane = threadIdx.x & 63;
  for (int64_t z = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6); z < Z; z += static_cast<int64_t>(gridDim.x) * 4) {
    // consecutive uses of one column j share a single reduction over the lanes (the caller may sort the uses by j)
    float acc = 0.f, p = 0.f;
    int cur = num_uses > 0 ? uses[0].j : 0;
    for (int u = 0; u < num_uses; ++u) {
      const FcDotUse use = uses[u];
      if (use.j != cur) {
        p = wave_sum(p);
        if (lane == cur) acc += p;
        p = 0.f;
        cur = use.j;
      }
      float q = 0.f;
      for (int k = lane; k < use.k; k += 64)
        q = fmaf(load_as<float>(X, type_code<TX>(), z * ldx + use.a_off + k), load_as<float>(G, type_code<TG>(), z * ldg + use.g_off + k), q);
      p = fmaf(use.coeff, q, p);
    }
    p = wave_sum(p);
    if (lane == cur) acc += p;
    if (lane < n2) store_as<float>(D, type_code<TX>(), z * ldd + lane, acc);
  }
}

// The same with four rows per wavefront: 16 lanes per row, four adjacent elements per lane (k, the offsets and the row
// strides are multiples of four); lane l of a row keeps the columns j = l, l + 16, l + 32, l + 48.
template <typename TX, typename TG>
__global__ void __launch_bounds__(256) fc_rowdot_vec_kernel(const TX* __restrict__ X, int64_t ldx, const TG* __restrict__ G, int64_t ldg,
                                                            TX* __restrict__ D, int64_t ldd, int n2, const FcDotUse* __restrict__ uses,
                                                            int num_uses, int64_t Z) {
  const int lane = threadIdx.x & 63, l16 = lane & 15, sub = lane >> 4;
  for (int64_t z0 = (static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6)) * 4; z0 < Z; z0 += static_cast<int64_t>(gridDim.x) * 16) {
    const int64_t z = min(z0 + sub, Z - 1);
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f, p = 0.f;
    int cur = num_uses > 0 ? uses[0].j : 0;
    auto commit = [&]() {
      p += __shfl_xor(p, 8, 64); p += __shfl_xor(p, 4, 64); p += __shfl_xor(p, 2, 64); p += __shfl_xor(p, 1, 64);
      if (l16 == (cur & 15)) {
        const int q = cur >> 4;
        if (q == 0) a0 += p; else if (q == 1) a1 += p; else if (q == 2) a2 += p; else a3 += p;
      }
      p = 0.f;
    };
    for (int u = 0; u < num_uses; ++u) {
      const FcDotUse use = uses[u];
      if (use.j != cur) { commit(); cur = use.j; }
      float q = 0.f;
      for (int k = 4 * l16; k < use.k; k += 64) {
        const float4 x = fc_load4(X + z * ldx + use.a_off + k), g = fc_load4(G + z * ldg + use.g_off + k);
        q = fmaf(x.x, g.x, q); q = fmaf(x.y, g.y, q); q = fmaf(x.z, g.z, q); q = fmaf(x.w, g.w, q);
      }
      p = fmaf(use.coeff, q, p);
    }
    commit();
    if (z0 + sub < Z) {
      if (l16 < n2) store_as<float>(D, type_code<TX>(), z * ldd + l16, a0);
      if (l16 + 16 < n2) store_as<float>(D, type_code<TX>(), z * ldd + l16 + 16, a1);
      if (l16 + 32 < n2) store_as<float>(D, type_code<TX>(), z * ldd + l16 + 32, a2);
      if (l16 + 48 < n2) store_as<float>(D, type_code<TX>(), z * ldd + l16 + 48, a3);
    }
  }
}

}  // namespace cueq

using namespace cueq;

extern "C" int cueq_seg_gemm(int32_t dtype, int32_t K, int32_t N, const void* A, int64_t lda, const void* B, const void* S,
                             int64_t lds_, void* C, int64_t ldc, int64_t rows, const cueq_gemm_problem* problems,
                             int32_t nproblems, int32_t force_simple, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(K > 0 && N > 0 && rows >= 0 && nproblems >= 0, CUEQ_ERR_INVALID, "bad sizes");
  CUEQ_REQUIRE(nproblems <= kMaxProblems, CUEQ_ERR_TOO_LARGE, "at most %d problems per call", kMaxProblems);
  static_assert(sizeof(GemmProblem) == sizeof(cueq_gemm_problem), "ABI struct mismatch");
  if (rows == 0 || nproblems == 0) return CUEQ_OK;
  CUEQ_REQUIRE(A && B && C && problems, CUEQ_ERR_INVALID, "null pointer");
  const GemmProblem* pp = reinterpret_cast<const GemmProblem*>(problems);
  const bool mfma_ok = (K == 32 || K == 64 || K == 128) && (N == 32 || N == 64 || N == 128) && (lda % 8 == 0);
  if (mfma_ok && !force_simple && (dtype == CUEQ_F32 || dtype == CUEQ_BF16)) {
    const int threads = 64 * (N / 32);
    const int rt = 1;
    const int64_t ntiles = (rows + 32 * rt - 1) / (32 * rt);
    int64_t gx = (static_cast<int64_t>(device_cus()) * 8 + nproblems - 1) / nproblems;
    if (gx > ntiles) gx = ntiles;
    if (gx < 1) gx = 1;
    const dim3 grid(static_cast<unsigned>(gx), static_cast<unsigned>(nproblems));
    KernelTimer timer(dtype == CUEQ_F32 ? "seg_gemm_f32" : "seg_gemm_bf16", stream);
    if (dtype == CUEQ_F32) {
      const size_t sh = 2 * 32 * (K + 4) * sizeof(float);
#define LAUNCH(KK, NW) hipLaunchKernelGGL((seg_gemm_f32<KK, NW, 1>), grid, dim3(threads), sh, stream, static_cast<const float*>(A), lda, static_cast<const float*>(B), static_cast<const float*>(S), lds_, static_cast<float*>(C), ldc, rows, N, pp)
#define LAUNCH_N(KK) switch (N) { case 32: LAUNCH(KK, 1); break; case 64: LAUNCH(KK, 2); break; default: LAUNCH(KK, 4); }
      switch (K) { case 32: LAUNCH_N(32); break; case 64: LAUNCH_N(64); break; default: LAUNCH_N(128); }
#undef LAUNCH_N
#undef LAUNCH
    } else {
      const size_t sh = 2 * 32 * (K + 8) * sizeof(uint16_t);
#define LAUNCH(KK, NW) hipLaunchKernelGGL((seg_gemm_bf16<KK, NW>), grid, dim3(threads), sh, stream, static_cast<const uint16_t*>(A), lda, static_cast<const uint16_t*>(B), static_cast<const uint16_t*>(S), lds_, static_cast<uint16_t*>(C), ldc, rows, N, pp)
#define LAUNCH_N(KK) switch (N) { case 32: LAUNCH(KK, 1); break; case 64: LAUNCH(KK, 2); break; default: LAUNCH(KK, 4); }
      switch (K) { case 32: LAUNCH_N(32); break; case 64: LAUNCH_N(64); break; default: LAUNCH_N(128); }
#undef LAUNCH_N
#undef LAUNCH
    }
    CUEQ_CHECK_HIP(hipGetLastError());
    return CUEQ_OK;
  }
  const int64_t total = rows * N;
  const dim3 grid(static_cast<unsigned>((total + 255) / 256), static_cast<unsigned>(nproblems));
  CUEQ_REQUIRE((total + 255) / 256 < (int64_t(1) << 31), CUEQ_ERR_TOO_LARGE, "too many rows");
  KernelTimer timer("seg_gemm_simple", stream);
  if (dtype == CUEQ_F32)
    hipLaunchKernelGGL((seg_gemm_simple<float, float>), grid, dim3(256), 0, stream, static_cast<const float*>(A), lda, static_cast<const float*>(B), static_cast<const float*>(S), lds_, static_cast<float*>(C), ldc, rows, K, N, pp);
  else if (dtype == CUEQ_F64)
    hipLaunchKernelGGL((seg_gemm_simple<double, double>), grid, dim3(256), 0, stream, static_cast<const double*>(A), lda, static_cast<const double*>(B), static_cast<const double*>(S), lds_, static_cast<double*>(C), ldc, rows, K, N, pp);
  else if (dtype == CUEQ_BF16)
    hipLaunchKernelGGL((seg_gemm_simple<uint16_t, float>), grid, dim3(256), 0, stream, static_cast<const uint16_t*>(A), lda, static_cast<const uint16_t*>(B), static_cast<const uint16_t*>(S), lds_, static_cast<uint16_t*>(C), ldc, rows, K, N, pp);
  else {
    set_error("seg_gemm: unsupported dtype %d", dtype);
    return CUEQ_ERR_UNSUPPORTED;
  }
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

static int64_t outer_slots(int64_t rows) {
  int64_t slots = static_cast<int64_t>(device_cus()) * 2;
  const int64_t max_by_rows = (rows + 255) / 256;  // at least 256 rows per slot
  if (slots > max_by_rows) slots = max_by_rows;
  return slots < 1 ? 1 : slots;
}

extern "C" int64_t cueq_seg_outer_workspace(int32_t dtype, int32_t K, int32_t N, int64_t rows) {
  const int64_t acc = dtype == CUEQ_F64 ? 8 : 4;
  return outer_slots(rows) * K * N * acc;
}

extern "C" int cueq_seg_outer(int32_t dtype, int32_t K, int32_t N, const void* A, int64_t lda, const void* G, int64_t ldg,
                              const void* S, int64_t lds_, void* dW, int64_t rows, const cueq_outer_entry* entries,
                              int32_t nentries, int32_t trans_out, int32_t accumulate, void* workspace,
                              int64_t workspace_bytes, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(K > 0 && N > 0 && rows >= 0 && nentries >= 1, CUEQ_ERR_INVALID, "bad sizes");
  static_assert(sizeof(OuterEntry) == sizeof(cueq_outer_entry), "ABI struct mismatch");
  CUEQ_REQUIRE(dW && entries && (rows == 0 || (A && G)), CUEQ_ERR_INVALID, "null pointer");
  (void)S;
  OuterProblem pr;
  pr.n_entries = nentries;
  pr.trans_out = trans_out;
  pr.e = reinterpret_cast<const OuterEntry*>(entries);
  const int64_t slots = outer_slots(rows);
  const int64_t need = cueq_seg_outer_workspace(dtype, K, N, rows);
  CUEQ_REQUIRE(workspace && workspace_bytes >= need, CUEQ_ERR_INVALID, "workspace too small: need %lld bytes", (long long)need);
  const int64_t rows_per_block = ((rows + slots - 1) / slots + 15) & ~int64_t(15);
  const int64_t kn = static_cast<int64_t>(K) * N;
  const bool mfma_ok = (K % 32 == 0) && K <= 256 && (N == 32 || N == 64 || N == 128) && (dtype == CUEQ_F32 || dtype == CUEQ_BF16);
  {
    KernelTimer timer(mfma_ok ? "seg_outer_mfma" : "seg_outer_simple", stream);
    if (mfma_ok) {
      const dim3 grid(static_cast<unsigned>(slots)), block(64 * (K / 32));
#define LAUNCH_OUTER(IO, NB) hipLaunchKernelGGL((seg_outer_mfma<IO, NB>), grid, block, 0, stream, static_cast<const IO*>(A), lda, static_cast<const IO*>(G), ldg, static_cast<const IO*>(S), lds_, static_cast<float*>(workspace), rows, K, rows_per_block, pr)
      if (dtype == CUEQ_F32) { switch (N) { case 32: LAUNCH_OUTER(float, 1); break; case 64: LAUNCH_OUTER(float, 2); break; default: LAUNCH_OUTER(float, 4); } }
      else { switch (N) { case 32: LAUNCH_OUTER(uint16_t, 1); break; case 64: LAUNCH_OUTER(uint16_t, 2); break; default: LAUNCH_OUTER(uint16_t, 4); } }
#undef LAUNCH_OUTER
    } else {
      const dim3 grid(static_cast<unsigned>((kn + 255) / 256), static_cast<unsigned>(slots));
      if (dtype == CUEQ_F32)
        hipLaunchKernelGGL((seg_outer_simple<float, float>), grid, dim3(256), 0, stream, static_cast<const float*>(A), lda, static_cast<const float*>(G), ldg, static_cast<const float*>(S), lds_, static_cast<float*>(workspace), rows, K, N, rows_per_block, pr);
      else if (dtype == CUEQ_F64)
        hipLaunchKernelGGL((seg_outer_simple<double, double>), grid, dim3(256), 0, stream, static_cast<const double*>(A), lda, static_cast<const double*>(G), ldg, static_cast<const double*>(S), lds_, static_cast<double*>(workspace), rows, K, N, rows_per_block, pr);
      else if (dtype == CUEQ_BF16)
        hipLaunchKernelGGL((seg_outer_simple<uint16_t, float>), grid, dim3(256), 0, stream, static_cast<const uint16_t*>(A), lda, static_cast<const uint16_t*>(G), ldg, static_cast<const uint16_t*>(S), lds_, static_cast<float*>(workspace), rows, K, N, rows_per_block, pr);
      else {
        set_error("seg_outer: unsupported dtype %d", dtype);
        return CUEQ_ERR_UNSUPPORTED;
      }
    }
  }
  CUEQ_CHECK_HIP(hipGetLastError());
  const dim3 fgrid(static_cast<unsigned>((kn + 255) / 256));
  if (dtype == CUEQ_F32)
    hipLaunchKernelGGL((fold_slots<float, float>), fgrid, dim3(256), 0, stream, static_cast<const float*>(workspace), static_cast<int>(slots), kn, static_cast<float*>(dW), accumulate);
  else if (dtype == CUEQ_F64)
    hipLaunchKernelGGL((fold_slots<double, double>), fgrid, dim3(256), 0, stream, static_cast<const double*>(workspace), static_cast<int>(slots), kn, static_cast<double*>(dW), accumulate);
  else
    hipLaunchKernelGGL((fold_slots<uint16_t, float>), fgrid, dim3(256), 0, stream, static_cast<const float*>(workspace), static_cast<int>(slots), kn, static_cast<uint16_t*>(dW), accumulate);
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

extern "C" int cueq_seg_rowdot(int32_t dtype, int32_t K, int32_t N, const void* A, int64_t lda, const void* B, const void* G,
                               int64_t ldg, void* dS, int64_t lds_, int64_t rows, const cueq_gemm_problem* problem,
                               void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(K > 0 && N > 0 && rows >= 0 && problem, CUEQ_ERR_INVALID, "bad arguments");
  if (rows == 0) return CUEQ_OK;
  CUEQ_REQUIRE(A && B && G && dS && problem->s_col >= 0, CUEQ_ERR_INVALID, "null pointer or missing scale column");
  const GemmProblem pr{problem->a_off, problem->c_off, problem->b_off, problem->alpha, problem->s_col, problem->trans_b,
                       problem->accumulate, 0};
  const dim3 grid(static_cast<unsigned>((rows * 64 + 255) / 256));
  if (dtype == CUEQ_F32)
    hipLaunchKernelGGL((seg_rowdot<float, float>), grid, dim3(256), 0, stream, static_cast<const float*>(A), lda, static_cast<const float*>(B), static_cast<const float*>(G), ldg, static_cast<float*>(dS), lds_, rows, K, N, pr);
  else if (dtype == CUEQ_F64)
    hipLaunchKernelGGL((seg_rowdot<double, double>), grid, dim3(256), 0, stream, static_cast<const double*>(A), lda, static_cast<const double*>(B), static_cast<const double*>(G), ldg, static_cast<double*>(dS), lds_, rows, K, N, pr);
  else if (dtype == CUEQ_BF16)
    hipLaunchKernelGGL((seg_rowdot<uint16_t, float>), grid, dim3(256), 0, stream, static_cast<const uint16_t*>(A), lda, static_cast<const uint16_t*>(B), static_cast<const uint16_t*>(G), ldg, static_cast<uint16_t*>(dS), lds_, rows, K, N, pr);
  else {
    set_error("seg_rowdot: unsupported dtype %d", dtype);
    return CUEQ_ERR_UNSUPPORTED;
  }
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

// dtype codes: s = x2 and the result (the tensor dtype), t = the GEMM results (float32 or the tensor dtype)
extern "C" int cueq_fc_combine(int32_t dtype, int32_t t_dtype, int64_t rows, const void* S, int64_t lds_, const void* T, int64_t ldt, void* O,
                               int64_t ldo, const void* blocks, int32_t num_blocks, const void* uses, int32_t max_n, int32_t vectorised,
                               void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE((dtype == CUEQ_F32 || dtype == CUEQ_BF16) && (t_dtype == CUEQ_F32 || t_dtype == dtype), CUEQ_ERR_UNSUPPORTED,
               "fc_combine: tensors float32 or bfloat16, GEMM results float32 or the tensor dtype");
  CUEQ_REQUIRE(rows >= 0 && num_blocks >= 0 && max_n >= 1 && max_n <= 256, CUEQ_ERR_INVALID, "fc_combine: bad extents (block width at most 256)");
  if (rows == 0 || num_blocks == 0) return CUEQ_OK;
  CUEQ_REQUIRE(S && T && O && blocks && uses, CUEQ_ERR_INVALID, "fc_combine: null operand");
  // four columns per thread when every block width, column offset and row stride is a multiple of four and the rows are
  // 16 / 8-byte aligned (the caller says so: it owns the tables)
  const bool vec = vectorised != 0 && max_n % 4 == 0 && ldt % 4 == 0 && ldo % 4 == 0 &&
                   reinterpret_cast<uintptr_t>(T) % 16 == 0 && reinterpret_cast<uintptr_t>(O) % 16 == 0;
  const int rpp = vec ? 256 / (max_n / 4) : 256 / max_n;
  int64_t gx = (rows + rpp - 1) / rpp;
  const int64_t cap = static_cast<int64_t>(device_cus()) * 32 / num_blocks + 1;
  if (gx > cap) gx = cap;
  const dim3 grid(static_cast<unsigned>(gx), static_cast<unsigned>(num_blocks));
  KernelTimer timer("fc_combine", stream);
  if (vec) {
#define FCV(TS, TT) hipLaunchKernelGGL((fc_combine_vec_kernel<TS, TT, TS>), grid, dim3(256), 0, stream, static_cast<const TS*>(S), lds_, static_cast<const TT*>(T), ldt, static_cast<TS*>(O), ldo, static_cast<const FcBlock*>(blocks), static_cast<const FcUse*>(uses), rows, max_n)
    if (dtype == CUEQ_F32) FCV(float, float);
    else if (t_dtype == CUEQ_F32) FCV(uint16_t, float);
    else FCV(uint16_t, uint16_t);
#undef FCV
    CUEQ_CHECK_HIP(hipGetLastError());
    return CUEQ_OK;
  }
#define FCC(TS, TT) hipLaunchKernelGGL((fc_combine_kernel<TS, TT, TS>), grid, dim3(256), 0, stream, static_cast<const TS*>(S), lds_, static_cast<const TT*>(T), ldt, static_cast<TS*>(O), ldo, static_cast<const FcBlock*>(blocks), static_cast<const FcUse*>(uses), rows, max_n)
  if (dtype == CUEQ_F32) FCC(float, float);
  else if (t_dtype == CUEQ_F32) FCC(uint16_t, float);
  else FCC(uint16_t, uint16_t);
#undef FCC
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

extern "C" int cueq_fc_rowdot(int32_t dtype, int32_t g_dtype, int64_t rows, const void* X, int64_t ldx, const void* G, int64_t ldg, void* D,
                              int64_t ldd, int32_t n2, const void* uses, int32_t num_uses, int32_t vectorised, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE((dtype == CUEQ_F32 || dtype == CUEQ_BF16) && (g_dtype == CUEQ_F32 || g_dtype == dtype), CUEQ_ERR_UNSUPPORTED,
               "fc_rowdot: tensors float32 or bfloat16, GEMM results float32 or the tensor dtype");
  CUEQ_REQUIRE(rows >= 0 && n2 >= 1 && n2 <= 64 && num_uses >= 0, CUEQ_ERR_UNSUPPORTED, "fc_rowdot: the multiplicity-one operand has at most 64 elements");
  if (rows == 0) return CUEQ_OK;
  CUEQ_REQUIRE(X && G && D && (uses || num_uses == 0), CUEQ_ERR_INVALID, "fc_rowdot: null operand");
  int64_t gx = (rows + 3) / 4;
  const int64_t cap = static_cast<int64_t>(device_cus()) * 32;
  if (gx > cap) gx = cap;
  KernelTimer timer("fc_rowdot", stream);
  // four elements per lane when the caller states that every k, a_off and g_off of the table is a multiple of four
  if (vectorised != 0 && ldx % 4 == 0 && ldg % 4 == 0 && reinterpret_cast<uintptr_t>(X) % 16 == 0 && reinterpret_cast<uintptr_t>(G) % 16 == 0) {
    int64_t gv = (rows + 15) / 16;
    if (gv > cap) gv = cap;
#define FCDV(TX, TG) hipLaunchKernelGGL((fc_rowdot_vec_kernel<TX, TG>), dim3(static_cast<unsigned>(gv)), dim3(256), 0, stream, static_cast<const TX*>(X), ldx, static_cast<const TG*>(G), ldg, static_cast<TX*>(D), ldd, n2, static_cast<const FcDotUse*>(uses), num_uses, rows)
    if (dtype == CUEQ_F32) FCDV(float, float);
    else if (g_dtype == CUEQ_F32) FCDV(uint16_t, float);
    else FCDV(uint16_t, uint16_t);
#undef FCDV
    CUEQ_CHECK_HIP(hipGetLastError());
    return CUEQ_OK;
  }
#define FCD(TX, TG) hipLaunchKernelGGL((fc_rowdot_kernel<TX, TG>), dim3(static_cast<unsigned>(gx)), dim3(256), 0, stream, static_cast<const TX*>(X), ldx, static_cast<const TG*>(G), ldg, static_cast<TX*>(D), ldd, n2, static_cast<const FcDotUse*>(uses), num_uses, rows)
  if (dtype == CUEQ_F32) FCD(float, float);
  else if (g_dtype == CUEQ_F32) FCD(uint16_t, float);
  else FCD(uint16_t, uint16_t);
#undef FCD
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}
