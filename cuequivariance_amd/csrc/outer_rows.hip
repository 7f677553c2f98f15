// Row-wise outer products of operand segments and their two contractions: the element-wise stage in front of the Linear map
// that evaluates the fully connected contraction u_v_uvw_w with a second operand of any multiplicity
// (FusedTensorProductOp4, cuequivariance_torch/cuequivariance_torch/primitives/segmented_polynomial_fused_tp.py:40-48, form
// list :114-129).  With the parts p = (a_off, b_off, p_off, na, nb) of a table,
//   outer:      P[z, p_off + u * nb + v] = A[z, a_off + u] * B[z, b_off + v]                      (a-major; b-major: p_off + v * na + u)
//   contract 0: O[z, seg_off + u] = sum over the parts p of the segment, in list order, and v of P[z, ..] * X[z, b_off_p + v]
//   contract 1: O[z, seg_off + v] = sum over the parts p of the segment, in list order, and u of P[z, ..] * X[z, a_off_p + u]
// The three are closed under differentiation (each one's gradients are the other two), so the stage is differentiable to any
// order on these kernels.  All of them are bound by the bytes of P: every element is written, or read, once; sums run in a
// fixed order (no atomics).  Elements of float64, float32, bfloat16 or half; the 2-byte types are multiplied and summed in
// float32 and rounded once.

#include "common.h"
#include "cw_common.h"
#include "u1d_spec.h"

namespace cueq {

struct OuterPart {
  int32_t a_off, b_off, p_off, na, nb;
};

// Element access: T is the type in memory (float, double, or the bits of a bfloat16 / half), Math<T> the type the products
// and sums are formed in (the same, or float for the 2-byte types: widened on load, rounded once on store).
template <typename T>
struct Math {
  typedef T type;
};
template <>
struct Math<uint16_t> {
  typedef float type;
};
template <>
struct Math<f16bits> {
  typedef float type;
};
template <typename T>
__device__ __forceinline__ typename Math<T>::type ld1(const T* p) {
  if constexpr (sizeof(T) == 2) return mm_widen<T>(*reinterpret_cast<const uint16_t*>(p));
  else return *p;
}
template <typename T>
__device__ __forceinline__ void st1(T* p, typename Math<T>::type v) {
  if constexpr (sizeof(T) == 2) *reinterpret_cast<uint16_t*>(p) = mm_round<T>(v);
  else *p = v;
}
// four adjacent elements (p on a boundary of four elements)
template <typename T>
__device__ __forceinline__ void ld4(const T* p, typename Math<T>::type (&v)[4]) {
  if constexpr (sizeof(T) == 2) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    v[0] = mm_widen<T>(static_cast<uint16_t>(w.x & 0xffffu)), v[1] = mm_widen<T>(static_cast<uint16_t>(w.x >> 16));
    v[2] = mm_widen<T>(static_cast<uint16_t>(w.y & 0xffffu)), v[3] = mm_widen<T>(static_cast<uint16_t>(w.y >> 16));
  } else if constexpr (sizeof(T) == 4) {
    const float4 w = *reinterpret_cast<const float4*>(p);
    v[0] = w.x, v[1] = w.y, v[2] = w.z, v[3] = w.w;
  } else {
    const double4 w = *reinterpret_cast<const double4*>(p);
    v[0] = w.x, v[1] = w.y, v[2] = w.z, v[3] = w.w;
  }
}
template <typename T>
__device__ __forceinline__ void st4(T* p, const typename Math<T>::type (&v)[4]) {
  if constexpr (sizeof(T) == 2) {
    uint2 w;
    w.x = static_cast<uint32_t>(mm_round<T>(v[0])) | (static_cast<uint32_t>(mm_round<T>(v[1])) << 16);
    w.y = static_cast<uint32_t>(mm_round<T>(v[2])) | (static_cast<uint32_t>(mm_round<T>(v[3])) << 16);
    *reinterpret_cast<uint2*>(p) = w;
  } else if constexpr (sizeof(T) == 4) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
    *reinterpret_cast<double4*>(p) = make_double4(v[0], v[1], v[2], v[3]);
  }
}

// V adjacent elements (p on a boundary of V elements); V = 8 is for the 2-byte types: one 16-byte access
template <typename T, int V>
__device__ __forceinline__ void ldv(const T* p, typename Math<T>::type (&v)[V]) {
  if constexpr (V == 8) {
    static_assert(sizeof(T) == 2, "eight elements at a time for 2-byte types only");
    const uint4 w = *reinterpret_cast<const uint4*>(p);
    const uint32_t words[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      v[2 * k] = mm_widen<T>(static_cast<uint16_t>(words[k] & 0xffffu));
      v[2 * k + 1] = mm_widen<T>(static_cast<uint16_t>(words[k] >> 16));
    }
  } else {
    ld4<T>(p, v);
  }
}
template <typename T, int V>
__device__ __forceinline__ void stv(T* p, const typename Math<T>::type (&v)[V]) {
  if constexpr (V == 8) {
    uint32_t words[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
      words[k] = static_cast<uint32_t>(mm_round<T>(v[2 * k])) | (static_cast<uint32_t>(mm_round<T>(v[2 * k + 1])) << 16);
    *reinterpret_cast<uint4*>(p) = make_uint4(words[0], words[1], words[2], words[3]);
  } else {
    st4<T>(p, v);
  }
}

// One part per blockIdx.y; a thread makes V adjacent elements of P for one row (V = 4 or 8: the fast index has an extent that
// is a multiple of V and every offset and row stride is too).
template <typename T, int V, bool AMAJOR>
__global__ void __launch_bounds__(256) outer_rows_kernel(const T* __restrict__ A, int64_t lda, const T* __restrict__ B, int64_t ldb,
                                                         T* __restrict__ P, int64_t ldp, const OuterPart* __restrict__ parts, int64_t rows) {
  const OuterPart part = parts[blockIdx.y];
  const int slow_n = AMAJOR ? part.na : part.nb, fast_n = AMAJOR ? part.nb : part.na;
  const int per_row = slow_n * (fast_n / V);
  const int64_t total = rows * per_row;
  for (int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; t < total; t += static_cast<int64_t>(gridDim.x) * 256) {
    const int64_t z = t / per_row;
    const int e = static_cast<int>(t - z * per_row);
    const int s = e / (fast_n / V), f = (e - s * (fast_n / V)) * V;
    const T* slow = AMAJOR ? A + z * lda + part.a_off : B + z * ldb + part.b_off;
    const T* fast = AMAJOR ? B + z * ldb + part.b_off : A + z * lda + part.a_off;
    T* out = P + z * ldp + part.p_off + static_cast<int64_t>(s) * fast_n + f;
    const typename Math<T>::type x = ld1<T>(slow + s);
    if constexpr (V > 1) {
      typename Math<T>::type y[V];
      ldv<T, V>(fast + f, y);
#pragma unroll
      for (int k = 0; k < V; ++k) y[k] *= x;
      stv<T, V>(out, y);
    } else {
      st1<T>(out, x * ld1<T>(fast + f));
    }
  }
}

// One output segment per blockIdx.y; a thread owns one element (row z, index i of the segment) and walks the parts of the
// segment and the contracted index.  WHICH = 0: the output carries the index of a, X is b; WHICH = 1: the reverse.  The
// contracted index is the fast one of P when (WHICH == 0) == AMAJOR: then the thread reads V adjacent elements at a time.
template <typename T, int V, int WHICH, bool AMAJOR>
__global__ void __launch_bounds__(256) outer_contract_kernel(const T* __restrict__ Q, int64_t ldq, const T* __restrict__ X, int64_t ldx,
                                                             T* __restrict__ O, int64_t ldo, const OuterPart* __restrict__ parts,
                                                             const int32_t* __restrict__ seg_start, const int32_t* __restrict__ seg_parts,
                                                             int64_t rows) {
  const int s = blockIdx.y;
  const int q0 = seg_start[s], q1 = seg_start[s + 1];
  if (q0 == q1) return;
  const OuterPart first = parts[seg_parts[q0]];
  const int n = WHICH == 0 ? first.na : first.nb;  // (all parts of a segment share the segment, hence its extent and offset)
  const int seg_off = WHICH == 0 ? first.a_off : first.b_off;
  constexpr bool kContractedIsFast = (WHICH == 0) == AMAJOR;
  const int64_t total = rows * n;
  for (int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; t < total; t += static_cast<int64_t>(gridDim.x) * 256) {
    const int64_t z = t / n;
    const int i = static_cast<int>(t - z * n);
    typedef typename Math<T>::type MT;
    MT acc = 0;
    for (int q = q0; q < q1; ++q) {
      const OuterPart part = parts[seg_parts[q]];
      const int m = WHICH == 0 ? part.nb : part.na;  // extent of the contracted index
      const T* x = X + z * ldx + (WHICH == 0 ? part.b_off : part.a_off);
      const T* p = Q + z * ldq + part.p_off;
      if constexpr (kContractedIsFast) {
        p += static_cast<int64_t>(i) * m;
        if constexpr (V > 1) {
          for (int k = 0; k < m; k += V) {
            MT a[V], b[V];
            ldv<T, V>(p + k, a);
            ldv<T, V>(x + k, b);
#pragma unroll
            for (int e = 0; e < V; ++e) acc += a[e] * b[e];
          }
        } else {
          for (int k = 0; k < m; ++k) acc += ld1<T>(p + k) * ld1<T>(x + k);
        }
      } else {
        p += i;  // the threads of a wavefront read adjacent elements
        for (int k = 0; k < m; ++k) acc += ld1<T>(p + static_cast<int64_t>(k) * n) * ld1<T>(x + k);
      }
    }
    st1<T>(O + z * ldo + seg_off + i, acc);
  }
}

static unsigned grid_for(int64_t items) {
  const int64_t cap = static_cast<int64_t>(device_cus()) * 64;
  int64_t blocks = (items + 255) / 256;
  if (blocks > cap) blocks = cap;
  return static_cast<unsigned>(blocks < 1 ? 1 : blocks);
}

static bool rows_aligned(const void* p, int64_t ld, int es, int v) {
  return reinterpret_cast<uintptr_t>(p) % (v * es) == 0 && ld % v == 0;
}

}  // namespace cueq

using namespace cueq;

extern "C" int cueq_outer_rows(int32_t dtype, int64_t rows, const void* A, int64_t lda, const void* B, int64_t ldb, void* P, int64_t ldp,
                               const void* parts, int32_t nparts, int32_t max_part, int32_t a_major, int32_t vectorised, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(dtype == CUEQ_F32 || dtype == CUEQ_F64 || dtype == CUEQ_BF16 || dtype == CUEQ_F16, CUEQ_ERR_UNSUPPORTED, "outer_rows: unknown dtype");
  CUEQ_REQUIRE(rows >= 0 && nparts >= 0 && nparts < 65536 && max_part >= 0 && lda >= 0 && ldb >= 0 && ldp >= 0, CUEQ_ERR_INVALID,
               "outer_rows: negative extent, or 65 536 parts and more");
  if (rows == 0 || nparts == 0 || max_part == 0) return CUEQ_OK;
  CUEQ_REQUIRE(A && B && P && parts, CUEQ_ERR_INVALID, "outer_rows: null operand");
  const int es = dtype_size(dtype);
  // vectorised: 0, or the number (4 or 8) that every offset and fast extent of the table is a multiple of
  const int v = (vectorised >= 8 && es == 2 && rows_aligned(A, lda, es, 8) && rows_aligned(B, ldb, es, 8) && rows_aligned(P, ldp, es, 8)) ? 8
                : (vectorised >= 4 && rows_aligned(A, lda, es, 4) && rows_aligned(B, ldb, es, 4) && rows_aligned(P, ldp, es, 4)) ? 4 : 1;
  const dim3 grid(grid_for(rows * (max_part / v)), static_cast<unsigned>(nparts));
  KernelTimer timer("outer_rows", stream);
#define LAUNCH(T, V, AM)                                                                                                        \
  hipLaunchKernelGGL((outer_rows_kernel<T, V, AM>), grid, dim3(256), 0, stream, static_cast<const T*>(A), lda, static_cast<const T*>(B), \
                     ldb, static_cast<T*>(P), ldp, static_cast<const OuterPart*>(parts), rows)
#define BY_ORDER(T, V) do { if (a_major) LAUNCH(T, V, true); else LAUNCH(T, V, false); } while (0)
#define BY_VEC(T) do { if (v == 4) BY_ORDER(T, 4); else BY_ORDER(T, 1); } while (0)
#define BY_VEC2(T) do { if (v == 8) BY_ORDER(T, 8); else BY_VEC(T); } while (0)
  if (dtype == CUEQ_F32) BY_VEC(float);
  else if (dtype == CUEQ_F64) BY_VEC(double);
  else if (dtype == CUEQ_BF16) BY_VEC2(uint16_t);
  else BY_VEC2(f16bits);
#undef BY_VEC2
#undef BY_VEC
#undef BY_ORDER
#undef LAUNCH
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

extern "C" int cueq_outer_rows_contract(int32_t dtype, int32_t which, int64_t rows, const void* Q, int64_t ldq, const void* X, int64_t ldx,
                                        void* O, int64_t ldo, const void* parts, const int32_t* seg_start, const int32_t* seg_parts,
                                        int32_t nsegs, int32_t max_extent, int32_t a_major, int32_t vectorised, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(dtype == CUEQ_F32 || dtype == CUEQ_F64 || dtype == CUEQ_BF16 || dtype == CUEQ_F16, CUEQ_ERR_UNSUPPORTED, "outer_rows_contract: unknown dtype");
  CUEQ_REQUIRE(which == 0 || which == 1, CUEQ_ERR_INVALID, "outer_rows_contract: which is 0 (sum over the index of b) or 1 (of a)");
  CUEQ_REQUIRE(rows >= 0 && nsegs >= 0 && nsegs < 65536 && max_extent >= 0 && ldq >= 0 && ldx >= 0 && ldo >= 0, CUEQ_ERR_INVALID,
               "outer_rows_contract: negative extent, or 65 536 segments and more");
  if (rows == 0 || nsegs == 0 || max_extent == 0) return CUEQ_OK;
  CUEQ_REQUIRE(Q && X && O && parts && seg_start && seg_parts, CUEQ_ERR_INVALID, "outer_rows_contract: null operand");
  const int es = dtype_size(dtype);
  const bool fast = (which == 0) == (a_major != 0);
  const int v = !fast ? 1
                : (vectorised >= 8 && es == 2 && rows_aligned(Q, ldq, es, 8) && rows_aligned(X, ldx, es, 8)) ? 8
                : (vectorised >= 4 && rows_aligned(Q, ldq, es, 4) && rows_aligned(X, ldx, es, 4)) ? 4 : 1;
  const dim3 grid(grid_for(rows * max_extent), static_cast<unsigned>(nsegs));
  KernelTimer timer("outer_rows_contract", stream);
#define LAUNCH(T, V, W, AM)                                                                                                        \
  hipLaunchKernelGGL((outer_contract_kernel<T, V, W, AM>), grid, dim3(256), 0, stream, static_cast<const T*>(Q), ldq,            \
                     static_cast<const T*>(X), ldx, static_cast<T*>(O), ldo, static_cast<const OuterPart*>(parts), seg_start, seg_parts, rows)
#define BY_SHAPE(T, V8)                                    \
  do {                                                     \
    if (which == 0 && a_major) {                           \
      if (v == 8) LAUNCH(T, V8, 0, true);                  \
      else if (v == 4) LAUNCH(T, 4, 0, true);              \
      else LAUNCH(T, 1, 0, true);                          \
    } else if (which == 0) LAUNCH(T, 1, 0, false);         \
    else if (a_major) LAUNCH(T, 1, 1, true);               \
    else if (v == 8) LAUNCH(T, V8, 1, false);              \
    else if (v == 4) LAUNCH(T, 4, 1, false);               \
    else LAUNCH(T, 1, 1, false);                           \
  } while (0)
  if (dtype == CUEQ_F32) BY_SHAPE(float, 4);
  else if (dtype == CUEQ_F64) BY_SHAPE(double, 4);
  else if (dtype == CUEQ_BF16) BY_SHAPE(uint16_t, 8);
  else BY_SHAPE(f16bits, 8);
#undef BY_SHAPE
#undef LAUNCH
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}
