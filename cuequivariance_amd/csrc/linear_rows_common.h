// Pieces shared by the row-streaming Linear launches (linear_rows.hip: rows with the channel index contiguous;
// linear_rows_mul_ir.hip: rows with the irrep component contiguous): the part table passed by value, 16-byte stream
// accesses, and the staging of the weight blocks into the local data share.
#pragma once

#include "common.h"

namespace cueq {
namespace {

typedef float lr_floatx16 __attribute__((ext_vector_type(16)));
typedef float lr_floatx2 __attribute__((ext_vector_type(2)));
typedef uint32_t lr_u32x4 __attribute__((ext_vector_type(4)));

// 16-byte accesses marked as streams: every byte of A and C is touched once
__device__ __forceinline__ uint4 lr_stream_load(const char* p) {
  const lr_u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const lr_u32x4*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void lr_stream_store(uint4 v, void* p) {
  const lr_u32x4 w = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(w, reinterpret_cast<lr_u32x4*>(p));
}

constexpr int kLrWaves = 8;
constexpr int kLrMaxParts = 48;
constexpr int kLrMaxSlots = 8;

struct LrPart {
  int32_t a_off, c_off, slot;
};
struct LrParts {
  LrPart part[kLrMaxParts];
  int64_t w_off[kLrMaxSlots];
};

// The weight blocks of a launch into LDS as rows of K elements (one row per result column, WRS bytes apart), 16-byte
// vectors requested in batches of four before the first is stored (one wait per batch instead of one per vector).
// w_contraction_major: the block lies K x N (a vector holds (k, n .. n + EPV - 1), which become column k of EPV rows);
// otherwise N x K, as the rows are wanted.  NTH threads take part.
template <typename TI, int NTH>
__device__ __forceinline__ void lr_stage_weights(const TI* __restrict__ W, const LrParts& parts, int nslots, int K, int N, int WRS,
                                                 int w_contraction_major, char* smem, int tid) {
  constexpr int ES = sizeof(TI), EPV = 16 / ES;
  for (int s = 0; s < nslots; ++s) {
    const TI* w = W + parts.w_off[s];
    char* dst = smem + s * (N * WRS);
    const int NVEC = K * N / EPV;  // vectors of the block
    for (int e0 = tid; e0 < NVEC; e0 += 4 * NTH) {
      uint4 v[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = *reinterpret_cast<const uint4*>(w + static_cast<int64_t>(e0 + j * NTH < NVEC ? e0 + j * NTH : e0) * EPV);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int e = e0 + j * NTH;
        if (e >= NVEC) continue;
        if (w_contraction_major) {
          const int k = e / (N / EPV), n = (e % (N / EPV)) * EPV;
          const uint32_t q[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
#pragma unroll
          for (int i = 0; i < EPV; ++i) {
            if constexpr (ES == 4) *reinterpret_cast<uint32_t*>(dst + (n + i) * WRS + 4 * k) = q[i];
            else *reinterpret_cast<uint16_t*>(dst + (n + i) * WRS + 2 * k) = static_cast<uint16_t>(q[i >> 1] >> (16 * (i & 1)));
          }
        } else {
          const int n = e / (K / EPV), vv = e % (K / EPV);
          *reinterpret_cast<uint4*>(dst + n * WRS + 16 * vv) = v[j];
        }
      }
    }
  }
}

}  // namespace
}  // namespace cueq
