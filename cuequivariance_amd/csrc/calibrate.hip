// Streaming micro-kernels that measure what the memory system of the device delivers to kernels shaped like the
// path-table kernels of this library (64-thread workgroups, one dword per lane and instruction, 8 wavefronts per CU):
// read, write, copy and floating-point atomic add over a caller-supplied buffer.  The roofline fractions the
// benchmark reports are against the published 8 TB/s; these figures say how much of it a kernel can reach at all
// (and that atomics run at one dword per clock and L2 channel, far below the streaming rates).

#include "common.h"
#include "u1d_spec.h"

namespace cueq {

template <int MODE>  // 0 read, 1 write, 2 atomic add, 3 copy
__global__ void __launch_bounds__(64) calibrate_kernel(const float* __restrict__ in, float* __restrict__ out, int64_t nrows, float* sink) {
  constexpr int NI = 32;  // dword instructions per row: a row is 32 x 64 floats = 8 KiB
  const int lane = threadIdx.x;
  float acc = 0;
  for (int64_t r = blockIdx.x; r < nrows; r += gridDim.x) {
    const float* ip = in + r * (NI * 64);
    float* op = out + r * (NI * 64);
    float v[NI];
    if (MODE == 0 || MODE == 3) {
#pragma unroll
      for (int i = 0; i < NI; ++i) v[i] = __builtin_nontemporal_load(ip + i * 64 + lane);
    } else {
#pragma unroll
      for (int i = 0; i < NI; ++i) v[i] = static_cast<float>(r + i);
    }
    if (MODE == 0) {
#pragma unroll
      for (int i = 0; i < NI; ++i) acc += v[i];
    }
    if (MODE == 1 || MODE == 3) {
#pragma unroll
      for (int i = 0; i < NI; ++i) __builtin_nontemporal_store(v[i], op + i * 64 + lane);
    }
    if (MODE == 2) {
#pragma unroll
      for (int i = 0; i < NI; ++i) unsafeAtomicAdd(op + i * 64 + lane, v[i]);
    }
  }
  if (acc == 12345.678f) *sink = acc;  // keeps the loads alive
}

}  // namespace cueq

using namespace cueq;

extern "C" int cueq_calibrate(int32_t kind, const void* in, void* out, int64_t bytes, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(kind >= 0 && kind <= 3, CUEQ_ERR_INVALID, "calibrate: kind must be 0 (read), 1 (write), 2 (atomic add) or 3 (copy)");
  CUEQ_REQUIRE(in && out && bytes >= 8192, CUEQ_ERR_INVALID, "calibrate: two buffers of at least 8 KiB are required");
  const int64_t nrows = bytes / 8192;
  int dev = 0;
  hipDeviceProp_t p;
  CUEQ_CHECK_HIP(hipGetDevice(&dev));
  CUEQ_CHECK_HIP(hipGetDeviceProperties(&p, dev));
  const unsigned grid = static_cast<unsigned>(p.multiProcessorCount) * 8;
  const float* a = static_cast<const float*>(in);
  float* b = static_cast<float*>(out);
  float* sink = b;  // never written: the guard value does not occur
  static const char* names[4] = {"calibrate_read", "calibrate_write", "calibrate_atomic", "calibrate_copy"};
  KernelTimer timer(names[kind], stream);
  switch (kind) {
    case 0: hipLaunchKernelGGL(calibrate_kernel<0>, dim3(grid), dim3(64), 0, stream, a, b, nrows, sink); break;
    case 1: hipLaunchKernelGGL(calibrate_kernel<1>, dim3(grid), dim3(64), 0, stream, a, b, nrows, sink); break;
    case 2: hipLaunchKernelGGL(calibrate_kernel<2>, dim3(grid), dim3(64), 0, stream, a, b, nrows, sink); break;
    default: hipLaunchKernelGGL(calibrate_kernel<3>, dim3(grid), dim3(64), 0, stream, a, b, nrows, sink); break;
  }
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}
