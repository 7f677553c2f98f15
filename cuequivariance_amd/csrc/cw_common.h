// Helpers shared by the generated channel-wise kernels: wavefront reductions and the small
// streaming kernels that finish a backward pass (row gather-sum, partial folding, zero fill).
#pragma once

#include "common.h"
#include "u1d_spec.h"

namespace cueq {

// ---- DPP lane exchange ------------------------------------------------------------------------
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, true));
}
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ double dpp_move(double v) {
  const uint64_t b = __builtin_bit_cast(uint64_t, v);
  const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(b & 0xffffffffu), CTRL, ROW_MASK, 0xf, true));
  const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(b >> 32), CTRL, ROW_MASK, 0xf, true));
  return __builtin_bit_cast(double, (static_cast<uint64_t>(hi) << 32) | lo);
}

// Sum over the 64 lanes, result valid in every lane.  Fixed butterfly: bit-reproducible.
template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
  v += dpp_move<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_move<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_move<0x141>(v);  // row_half_mirror
  v += dpp_move<0x140>(v);  // row_mirror: every lane holds its row's sum
  v += __shfl_xor(v, 16, 64);
  v += __shfl_xor(v, 32, 64);
  return v;
}

// ---- element types of the buffers ----------------------------------------------------------------
// The generated kernels compute in `float` or `double`; their buffers hold that type or, for `float` arithmetic, 16-bit
// elements (bfloat16 as its bits, IEEE half) that are widened when loaded and rounded to nearest even when stored.
struct bf16_t { uint16_t bits; };
using f16_t = _Float16;

template <typename TI> struct math_of { using type = TI; };  // the arithmetic type that goes with an element type
template <> struct math_of<bf16_t> { using type = float; };
template <> struct math_of<f16_t> { using type = float; };

template <typename T> struct dtype_code;
template <> struct dtype_code<float> { static constexpr int value = CUEQ_F32; };
template <> struct dtype_code<double> { static constexpr int value = CUEQ_F64; };
template <> struct dtype_code<bf16_t> { static constexpr int value = CUEQ_BF16; };
template <> struct dtype_code<f16_t> { static constexpr int value = CUEQ_F16; };

__device__ __forceinline__ float io_ld(const float* p) { return *p; }
__device__ __forceinline__ double io_ld(const double* p) { return *p; }
__device__ __forceinline__ float io_ld(const bf16_t* p) { return bf16_bits_to_float(p->bits); }
__device__ __forceinline__ float io_ld(const f16_t* p) { return static_cast<float>(*p); }
__device__ __forceinline__ void io_st(float v, float* p) { *p = v; }
__device__ __forceinline__ void io_st(double v, double* p) { *p = v; }
// (float -> bfloat16: the hardware's conversion, round to nearest even, one instruction)
__device__ __forceinline__ uint16_t io_bf16_bits(float v) { return __builtin_bit_cast(uint16_t, static_cast<__bf16>(v)); }
__device__ __forceinline__ void io_st(float v, bf16_t* p) { p->bits = io_bf16_bits(v); }
__device__ __forceinline__ void io_st(float v, f16_t* p) { *p = static_cast<f16_t>(v); }
// the same for data read or written once per launch (non-temporal: they do not displace gathered rows in the caches)
#ifndef CUEQ_CW_NO_STREAM
__device__ __forceinline__ float io_ldnt(const float* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ double io_ldnt(const double* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ float io_ldnt(const bf16_t* p) { return bf16_bits_to_float(__builtin_nontemporal_load(&p->bits)); }
__device__ __forceinline__ float io_ldnt(const f16_t* p) { return static_cast<float>(__builtin_nontemporal_load(p)); }
__device__ __forceinline__ void io_stnt(float v, float* p) { __builtin_nontemporal_store(v, p); }
__device__ __forceinline__ void io_stnt(double v, double* p) { __builtin_nontemporal_store(v, p); }
__device__ __forceinline__ void io_stnt(float v, bf16_t* p) { __builtin_nontemporal_store(io_bf16_bits(v), &p->bits); }
__device__ __forceinline__ void io_stnt(float v, f16_t* p) { __builtin_nontemporal_store(static_cast<f16_t>(v), p); }
#else
template <typename TI> __device__ __forceinline__ auto io_ldnt(const TI* p) { return io_ld(p); }
template <typename M, typename TI> __device__ __forceinline__ void io_stnt(M v, TI* p) { io_st(v, p); }
#endif

// the element type shared by buffers [0, n), as a CUEQ_* code, or -1 when they differ
inline int common_dtype(const cueq_u1d_buffer* b, int n) {
  for (int i = 1; i < n; ++i) if (b[i].dtype != b[0].dtype) return -1;
  return b[0].dtype;
}

// out[i] = in[i] rounded to TO (the gradient of a gathered operand is summed in the arithmetic type and rounded once)
template <typename M, typename TO>
__global__ void __launch_bounds__(256) round_rows(const M* __restrict__ in, int64_t n, TO* __restrict__ out) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) io_st(in[i], out + i);
}

// ---- finishing kernels ------------------------------------------------------------------------
// out[r, :] = sum over zz in [offsets[r], offsets[r+1]) of partial[perm[zz], :]   (width elements per row)
template <typename T>
__global__ void __launch_bounds__(256) segment_sum_rows(const T* __restrict__ partial, const int64_t* __restrict__ offsets,
                                                        const int64_t* __restrict__ perm, int64_t nrows, int width,
                                                        T* __restrict__ out) {
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t r = tid / width;
  if (r >= nrows) return;
  const int c = static_cast<int>(tid - r * width);
  typename math_of<T>::type acc = 0;
  for (int64_t zz = offsets[r]; zz < offsets[r + 1]; ++zz) acc += io_ld(partial + perm[zz] * width + c);
  io_st(acc, out + tid);
}

// The same sum for rows whose width is a multiple of 4 elements (16-byte aligned rows): a thread owns 4 consecutive
// columns, the row ids of 8 contributions are read ahead and their 8 loads are in flight together; the additions keep the
// order of the list, so the result is the same from run to run.  One block of 256 threads per 1024 columns of a row.
template <typename T>
__global__ void __launch_bounds__(256) segment_sum_rows_vec(const T* __restrict__ partial, const int64_t* __restrict__ offsets,
                                                            const int64_t* __restrict__ perm, int width, T* __restrict__ out) {
  struct alignas(4 * sizeof(T)) V4 { T v[4]; };
  const int64_t r = blockIdx.y;
  const int c = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (c >= width) return;
  const int64_t z0 = offsets[r], z1 = offsets[r + 1];
  typename math_of<T>::type acc[4] = {0, 0, 0, 0};
  int64_t zz = z0;
  for (; zz + 8 <= z1; zz += 8) {
    V4 x[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) x[k] = *reinterpret_cast<const V4*>(partial + perm[zz + k] * width + c);
#pragma unroll
    for (int k = 0; k < 8; ++k)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] += io_ld(&x[k].v[e]);
  }
  for (; zz < z1; ++zz) {
    const V4 x = *reinterpret_cast<const V4*>(partial + perm[zz] * width + c);
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] += io_ld(&x.v[e]);
  }
  V4 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) io_st(acc[e], &o.v[e]);
  *reinterpret_cast<V4*>(out + r * width + c) = o;
}

// out[z, j] = sum over c in [0, nparts) of partial[(z * nparts + c), j]   (partials in the arithmetic type)
template <typename T, typename TO = T>
__global__ void __launch_bounds__(256) fold_parts(const T* __restrict__ partial, int64_t n, int nparts, int width,
                                                  TO* __restrict__ out) {
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tid >= n * width) return;
  const int64_t z = tid / width;
  const int j = static_cast<int>(tid - z * width);
  T acc = 0;
  for (int c = 0; c < nparts; ++c) acc += partial[(z * nparts + c) * width + j];
  io_st(acc, out + tid);
}

// p[0 .. n) = 0, 16 bytes per thread (element by element when p is not 16-byte aligned, and for the tail);
// launch with fill_blocks<T>(n) blocks of 256 threads
template <typename T>
__global__ void __launch_bounds__(256) fill_zero(T* __restrict__ p, int64_t n) {
  constexpr int V = 16 / sizeof(T);
  const int64_t i = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * V;
  if (i >= n) return;
  if (i + V <= n && reinterpret_cast<uintptr_t>(p) % 16 == 0) {
    *reinterpret_cast<uint4*>(p + i) = make_uint4(0u, 0u, 0u, 0u);
  } else {
    for (int64_t k = i; k < n && k < i + V; ++k) p[k] = T{};
  }
}

template <typename T>
inline unsigned fill_blocks(int64_t n) {
  constexpr int V = 16 / sizeof(T);
  const int64_t threads = (n + V - 1) / V;
  return static_cast<unsigned>((threads + 255) / 256);
}

// Compute units of the current device (cached for the first device queried).
inline int device_cus() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t p;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) cus = p.multiProcessorCount;
    if (cus <= 0) cus = 256;
  }
  return cus;
}

// Number of resident wavefront slots to fill: compute units x 4 SIMDs x waves per SIMD.
inline int64_t wave_slots(int waves_per_simd) { return static_cast<int64_t>(device_cus()) * 4 * waves_per_simd; }

inline unsigned blocks_for(int64_t n, int per_block = 256) { return static_cast<unsigned>((n + per_block - 1) / per_block); }

// Scatter policy of the fused backward for the gradient of a gathered operand:
// hardware floating-point atomics (fast, summation order varies) or per-row partials
// followed by a gather-sum in index order (bit-reproducible, one extra pass over batch x row).
// A process-wide option (cueq_set_option("deterministic", ...); initial value from CUEQ_DETERMINISTIC, read once).
bool deterministic_scatter();

}  // namespace cueq
