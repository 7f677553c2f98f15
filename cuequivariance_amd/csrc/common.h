// Shared helpers for the gfx950 kernels: error reporting across the C ABI and
// element load/store with conversion between the tensor dtype and the math dtype.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "cueq_amd.h"

namespace cueq {

void set_error(const char* fmt, ...);

#define CUEQ_CHECK_HIP(expr)                                                              \
  do {                                                                                    \
    hipError_t _e = (expr);                                                               \
    if (_e != hipSuccess) {                                                               \
      ::cueq::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__,  \
                        __LINE__);                                                        \
      return CUEQ_ERR_HIP;                                                                \
    }                                                                                     \
  } while (0)

#define CUEQ_REQUIRE(cond, code, ...)  \
  do {                                 \
    if (!(cond)) {                     \
      ::cueq::set_error(__VA_ARGS__);  \
      return (code);                   \
    }                                  \
  } while (0)

__host__ __device__ inline int dtype_size(int dt) {
  return dt == CUEQ_F64 ? 8 : (dt == CUEQ_F32 ? 4 : 2);
}

// ---- 2-byte element formats of the matrix-core kernels ---------------------------------------------------------------
// Those kernels move 2-byte elements as words; only the product instruction and the rounding of results depend on the
// format.  The element type selects it: uint16_t = bfloat16 (as its bits), f16bits = IEEE half (as its bits).
struct f16bits { uint16_t bits; };
typedef float mm_floatx16 __attribute__((ext_vector_type(16)));
typedef float mm_floatx4 __attribute__((ext_vector_type(4)));
typedef float mm_floatx2 __attribute__((ext_vector_type(2)));
typedef __bf16 mm_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 mm_bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 mm_f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 mm_f16x2 __attribute__((ext_vector_type(2)));
template <typename TI> struct is_half_bits { static constexpr bool value = false; };
template <> struct is_half_bits<f16bits> { static constexpr bool value = true; };

// acc += A (32 x 16) B (16 x 32), eight 2-byte elements per lane and operand
template <typename TI>
__device__ __forceinline__ mm_floatx16 mm_32x32x16(uint4 a, uint4 b, mm_floatx16 acc) {
  if constexpr (is_half_bits<TI>::value)
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(mm_f16x8, a), __builtin_bit_cast(mm_f16x8, b), acc, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(mm_bf16x8, a), __builtin_bit_cast(mm_bf16x8, b), acc, 0, 0, 0);
}
// acc += A (16 x 32) B (32 x 16)
template <typename TI>
__device__ __forceinline__ mm_floatx4 mm_16x16x32(uint4 a, uint4 b, mm_floatx4 acc) {
  if constexpr (is_half_bits<TI>::value)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(mm_f16x8, a), __builtin_bit_cast(mm_f16x8, b), acc, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(mm_bf16x8, a), __builtin_bit_cast(mm_bf16x8, b), acc, 0, 0, 0);
}
// two floats rounded to nearest even and packed, `lo` in the low half (one conversion instruction)
template <typename TI>
__device__ __forceinline__ uint32_t mm_pack(float lo, float hi) {
  const mm_floatx2 f = {lo, hi};
  if constexpr (is_half_bits<TI>::value) return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, mm_f16x2));
  else return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, mm_bf16x2));
}
// one element widened to float / one float rounded to the format
template <typename TI>
__device__ __forceinline__ float mm_widen(uint16_t bits) {
  if constexpr (is_half_bits<TI>::value) return static_cast<float>(__builtin_bit_cast(_Float16, bits));
  else return __uint_as_float(static_cast<uint32_t>(bits) << 16);
}
template <typename TI>
__device__ __forceinline__ uint16_t mm_round(float v) {
  if constexpr (is_half_bits<TI>::value) return __builtin_bit_cast(uint16_t, static_cast<_Float16>(v));
  else return __builtin_bit_cast(uint16_t, static_cast<__bf16>(v));
}

// bf16 <-> f32 by bit manipulation (round to nearest even on the way down).
__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) {
  return __uint_as_float(static_cast<uint32_t>(b) << 16);
}
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  uint32_t x = __float_as_uint(f);
  if ((x & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((x >> 16) | 0x40u);  // quiet NaN
  x += 0x7fffu + ((x >> 16) & 1u);
  return static_cast<uint16_t>(x >> 16);
}

template <typename M>
__device__ __forceinline__ M load_as(const void* p, int dt, int64_t i) {
  switch (dt) {
    case CUEQ_F32: return static_cast<M>(static_cast<const float*>(p)[i]);
    case CUEQ_F64: return static_cast<M>(static_cast<const double*>(p)[i]);
    case CUEQ_F16: return static_cast<M>(__half2float(static_cast<const __half*>(p)[i]));
    default: return static_cast<M>(bf16_bits_to_float(static_cast<const uint16_t*>(p)[i]));
  }
}

template <typename M>
__device__ __forceinline__ void store_as(void* p, int dt, int64_t i, M v) {
  switch (dt) {
    case CUEQ_F32: static_cast<float*>(p)[i] = static_cast<float>(v); break;
    case CUEQ_F64: static_cast<double*>(p)[i] = static_cast<double>(v); break;
    case CUEQ_F16: static_cast<__half*>(p)[i] = __float2half(static_cast<float>(v)); break;
    default: static_cast<uint16_t*>(p)[i] = float_to_bf16_bits(static_cast<float>(v)); break;
  }
}

__device__ __forceinline__ int64_t load_index(const void* p, int is64, int64_t i) {
  return is64 ? static_cast<const int64_t*>(p)[i] : static_cast<int64_t>(static_cast<const int32_t*>(p)[i]);
}

}  // namespace cueq
