// Per-segment (u, v) -> (v, u) transposition of every row of a 2-D tensor in one pass: the layout change between
// mul_ir and ir_mul.  Stands for the reference's native op behind
// cuequivariance_torch/cuequivariance_torch/primitives/transpose.py:83-183 (segmented_transpose).
//
// The permutation of a row is the same for all rows, so the host passes it as a table src[o] = input position of
// output element o.  A block moves one row: coalesced read into LDS, permuted read out of LDS, coalesced write.  Rows
// too long for LDS are gathered straight from global memory.

#include "common.h"
#include "cw_common.h"
#include "u1d_spec.h"

namespace cueq {

constexpr int kSegTransposeLdsBytes = 48 * 1024;

template <typename T, bool USE_LDS>
__global__ void __launch_bounds__(256) segmented_transpose_kernel(const T* __restrict__ in, T* __restrict__ out, const int32_t* __restrict__ src,
                                                                  int64_t rows, int total) {
  extern __shared__ __align__(16) char seg_lds[];
  T* row = reinterpret_cast<T*>(seg_lds);
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    const T* x = in + r * total;
    T* y = out + r * total;
    if constexpr (USE_LDS) {
      __syncthreads();  // the previous row is no longer read
      for (int i = threadIdx.x; i < total; i += 256) row[i] = x[i];
      __syncthreads();
      for (int o = threadIdx.x; o < total; o += 256) y[o] = row[src[o]];
    } else {
      for (int o = threadIdx.x; o < total; o += 256) y[o] = x[src[o]];
    }
  }
}

}  // namespace cueq

using namespace cueq;

extern "C" int cueq_segmented_transpose(int32_t element_size, int64_t rows, int64_t total, const int32_t* src_index, const void* in, void* out,
                                        void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(element_size == 2 || element_size == 4 || element_size == 8, CUEQ_ERR_UNSUPPORTED, "segmented_transpose: element size must be 2, 4 or 8 bytes");
  CUEQ_REQUIRE(rows >= 0 && total >= 0 && total < (1ll << 31), CUEQ_ERR_INVALID, "segmented_transpose: bad extents");
  if (rows == 0 || total == 0) return CUEQ_OK;
  CUEQ_REQUIRE(src_index && in && out, CUEQ_ERR_INVALID, "segmented_transpose: null operand");
  CUEQ_REQUIRE(in != out, CUEQ_ERR_INVALID, "segmented_transpose: cannot run in place");
  const int64_t cap = static_cast<int64_t>(device_cus()) * 16;
  const unsigned grid = static_cast<unsigned>(rows < cap ? rows : cap);
  const size_t lds = static_cast<size_t>(total) * element_size;
  const bool use_lds = lds <= static_cast<size_t>(kSegTransposeLdsBytes);
  KernelTimer timer("segmented_transpose", stream);
#define ST(T) do { if (use_lds) hipLaunchKernelGGL((segmented_transpose_kernel<T, true>), dim3(grid), dim3(256), lds, stream, static_cast<const T*>(in), static_cast<T*>(out), src_index, rows, static_cast<int>(total)); \
                   else hipLaunchKernelGGL((segmented_transpose_kernel<T, false>), dim3(grid), dim3(256), 0, stream, static_cast<const T*>(in), static_cast<T*>(out), src_index, rows, static_cast<int>(total)); } while (0)
  if (element_size == 2) ST(uint16_t);
  else if (element_size == 4) ST(uint32_t);
  else ST(uint64_t);
#undef ST
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}
