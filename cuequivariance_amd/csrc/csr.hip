// Grouping of batch rows by the output row they scatter into.
//
// The scatter-add of an indexed output (reference:
// cuequivariance_torch/cuequivariance_torch/primitives/segmented_polynomial_naive.py:409-418)
// is turned into a gather: perm lists the batch ids sorted by output row (stable, so ids
// ascend inside a row) and offsets[r] .. offsets[r+1] delimits row r.  The executor then sums
// each row's contributions in that fixed order, which makes the result independent of
// scheduling.  Already-sorted ids (the common "receivers sorted" case) skip the sort.

#include <hipcub/hipcub.hpp>

#include "common.h"

namespace cueq {

__global__ void __launch_bounds__(256) csr_load_keys(const void* index, int is64, int64_t n, int64_t nrows,
                                                     uint32_t* keys, uint32_t* iota, int* flags) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int64_t v = load_index(index, is64, i);
  if (v < 0 || v >= nrows) flags[0] = 1;  // out of range
  if (i > 0 && load_index(index, is64, i - 1) > v) flags[1] = 1;  // not sorted
  keys[i] = static_cast<uint32_t>(v);
  iota[i] = static_cast<uint32_t>(i);
}

// offsets[r] = number of keys < r  (keys sorted ascending), r in [0, nrows]
__global__ void __launch_bounds__(256) csr_offsets(const uint32_t* sorted_keys, int64_t n, int64_t nrows,
                                                   int64_t* offsets) {
  const int64_t r = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (r > nrows) return;
  int64_t lo = 0, hi = n;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (static_cast<int64_t>(sorted_keys[mid]) < r) lo = mid + 1; else hi = mid;
  }
  offsets[r] = lo;
}

__global__ void __launch_bounds__(256) csr_widen(const uint32_t* src, int64_t n, int64_t* dst) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

// Capture-safe variant of csr_load_keys: nothing is reported to the host; ids outside [0, nrows) get the key nrows, so
// they sort behind every row and no row's range includes them.
__global__ void __launch_bounds__(256) csr_load_keys_clamped(const void* index, int is64, int64_t n, int64_t nrows,
                                                             uint32_t* keys, uint32_t* iota) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int64_t v = load_index(index, is64, i);
  keys[i] = static_cast<uint32_t>((v < 0 || v >= nrows) ? nrows : v);
  iota[i] = static_cast<uint32_t>(i);
}

__global__ void __launch_bounds__(256) csr_zero_offsets(int64_t* offsets, int64_t count) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < count) offsets[i] = 0;
}

static size_t sort_temp_bytes(int64_t n) {
  size_t bytes = 0;
  hipcub::DeviceRadixSort::SortPairs(nullptr, bytes, static_cast<const uint32_t*>(nullptr),
                                     static_cast<uint32_t*>(nullptr), static_cast<const uint32_t*>(nullptr),
                                     static_cast<uint32_t*>(nullptr), static_cast<int>(n));
  return bytes;
}

static size_t align256(size_t x) { return (x + 255) & ~size_t(255); }

}  // namespace cueq

using namespace cueq;

extern "C" int64_t cueq_segment_csr_workspace(int64_t n, int64_t nrows) {
  (void)nrows;
  if (n <= 0) return 256;
  // keys, iota, sorted keys, sorted iota, flags, radix-sort temporaries
  return static_cast<int64_t>(4 * align256(n * sizeof(uint32_t)) + 256 + align256(sort_temp_bytes(n)));
}

extern "C" int cueq_segment_csr_build(const void* index, int32_t index_is_64, int64_t n, int64_t nrows,
                                      int64_t* offsets, int64_t* perm, void* workspace, int64_t workspace_bytes,
                                      void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(n >= 0 && nrows >= 0 && offsets, CUEQ_ERR_INVALID, "bad arguments");
  CUEQ_REQUIRE(n < (int64_t(1) << 31) && nrows < (int64_t(1) << 31), CUEQ_ERR_TOO_LARGE,
               "at most 2^31-1 ids / rows are supported");
  if (n == 0) {
    hipLaunchKernelGGL(csr_zero_offsets, dim3(static_cast<unsigned>((nrows + 1 + 255) / 256)), dim3(256), 0, stream, offsets, nrows + 1);
    CUEQ_CHECK_HIP(hipGetLastError());
    return CUEQ_OK;
  }
  CUEQ_REQUIRE(index && perm && workspace, CUEQ_ERR_INVALID, "null pointer");
  CUEQ_REQUIRE(workspace_bytes >= cueq_segment_csr_workspace(n, nrows), CUEQ_ERR_INVALID, "workspace too small");
  char* w = static_cast<char*>(workspace);
  const size_t a = align256(n * sizeof(uint32_t));
  auto* keys = reinterpret_cast<uint32_t*>(w);
  auto* iota = reinterpret_cast<uint32_t*>(w + a);
  auto* skeys = reinterpret_cast<uint32_t*>(w + 2 * a);
  auto* siota = reinterpret_cast<uint32_t*>(w + 3 * a);
  auto* flags = reinterpret_cast<int*>(w + 4 * a);
  void* temp = w + 4 * a + 256;
  size_t temp_bytes = sort_temp_bytes(n);

  const unsigned nb = static_cast<unsigned>((n + 255) / 256);
  hipLaunchKernelGGL(csr_zero_offsets, dim3(1), dim3(256), 0, stream, reinterpret_cast<int64_t*>(flags), 1);  // both flags
  CUEQ_CHECK_HIP(hipGetLastError());
  hipLaunchKernelGGL(csr_load_keys, dim3(nb), dim3(256), 0, stream, index, index_is_64, n, nrows, keys, iota, flags);
  CUEQ_CHECK_HIP(hipGetLastError());
  int h_flags[2] = {0, 0};
  CUEQ_CHECK_HIP(hipMemcpyAsync(h_flags, flags, sizeof(h_flags), hipMemcpyDeviceToHost, stream));
  CUEQ_CHECK_HIP(hipStreamSynchronize(stream));
  CUEQ_REQUIRE(h_flags[0] == 0, CUEQ_ERR_INVALID, "index out of range [0, %lld)", (long long)nrows);
  const uint32_t* final_keys = keys;
  const uint32_t* final_perm = iota;
  if (h_flags[1]) {
    int end_bit = 1;
    while ((int64_t(1) << end_bit) < nrows && end_bit < 32) ++end_bit;
    CUEQ_CHECK_HIP(hipcub::DeviceRadixSort::SortPairs(temp, temp_bytes, keys, skeys, iota, siota, static_cast<int>(n),
                                                      0, end_bit, stream));
    final_keys = skeys;
    final_perm = siota;
  }
  const unsigned nbr = static_cast<unsigned>((nrows + 1 + 255) / 256);
  hipLaunchKernelGGL(csr_offsets, dim3(nbr), dim3(256), 0, stream, final_keys, n, nrows, offsets);
  CUEQ_CHECK_HIP(hipGetLastError());
  hipLaunchKernelGGL(csr_widen, dim3(nb), dim3(256), 0, stream, final_perm, n, perm);
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}

// The same grouping with device-side work only: no host read of the "sorted" / "in range" flags, no memset node, so the
// call may be recorded into a HIP graph and regroups from the live index buffer on every replay.  Always sorts
// (stable radix sort, so already-sorted ids come out unchanged).  Ids outside [0, nrows) cannot be reported from
// here: they are left out of every row's range.
extern "C" int cueq_segment_csr_build_async(const void* index, int32_t index_is_64, int64_t n, int64_t nrows,
                                            int64_t* offsets, int64_t* perm, void* workspace, int64_t workspace_bytes,
                                            void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(n >= 0 && nrows >= 0 && offsets, CUEQ_ERR_INVALID, "bad arguments");
  CUEQ_REQUIRE(n < (int64_t(1) << 31) && nrows < (int64_t(1) << 31) - 1, CUEQ_ERR_TOO_LARGE,
               "at most 2^31-1 ids / 2^31-2 rows are supported");
  if (n == 0) {
    hipLaunchKernelGGL(csr_zero_offsets, dim3(static_cast<unsigned>((nrows + 1 + 255) / 256)), dim3(256), 0, stream, offsets, nrows + 1);
    CUEQ_CHECK_HIP(hipGetLastError());
    return CUEQ_OK;
  }
  CUEQ_REQUIRE(index && perm && workspace, CUEQ_ERR_INVALID, "null pointer");
  CUEQ_REQUIRE(workspace_bytes >= cueq_segment_csr_workspace(n, nrows), CUEQ_ERR_INVALID, "workspace too small");
  char* w = static_cast<char*>(workspace);
  const size_t a = align256(n * sizeof(uint32_t));
  auto* keys = reinterpret_cast<uint32_t*>(w);
  auto* iota = reinterpret_cast<uint32_t*>(w + a);
  auto* skeys = reinterpret_cast<uint32_t*>(w + 2 * a);
  auto* siota = reinterpret_cast<uint32_t*>(w + 3 * a);
  void* temp = w + 4 * a + 256;
  size_t temp_bytes = sort_temp_bytes(n);
  const unsigned nb = static_cast<unsigned>((n + 255) / 256);
  hipLaunchKernelGGL(csr_load_keys_clamped, dim3(nb), dim3(256), 0, stream, index, index_is_64, n, nrows, keys, iota);
  CUEQ_CHECK_HIP(hipGetLastError());
  int end_bit = 1;
  while ((int64_t(1) << end_bit) <= nrows && end_bit < 32) ++end_bit;  // keys reach nrows (the out-of-range key)
  CUEQ_CHECK_HIP(hipcub::DeviceRadixSort::SortPairs(temp, temp_bytes, keys, skeys, iota, siota, static_cast<int>(n), 0, end_bit, stream));
  const unsigned nbr = static_cast<unsigned>((nrows + 1 + 255) / 256);
  hipLaunchKernelGGL(csr_offsets, dim3(nbr), dim3(256), 0, stream, skeys, n, nrows, offsets);
  CUEQ_CHECK_HIP(hipGetLastError());
  hipLaunchKernelGGL(csr_widen, dim3(nb), dim3(256), 0, stream, siota, n, perm);
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}
