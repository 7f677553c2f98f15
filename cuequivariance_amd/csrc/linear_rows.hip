// Row-streaming product for Linear-like operations (bfloat16 or float32 elements, float32 accumulation):
//   C[z, c_p : c_p + N] = alpha * A[z, a_p : a_p + K] * W_s(p)      for every part p of a host table, all rows z,
// with every distinct weight block W_s resident in LDS for the whole launch.  One persistent block per compute unit;
// each wavefront walks units (32 rows, part) on its own: the rows of A are requested ahead (bfloat16: three units, in
// three rotating register sets; float32: one) as they lie in memory (every load instruction covers whole 128-byte pieces of rows), pass through a staging tile private to the
// wavefront to become MFMA operands, the weight fragments come from LDS, and the 32 x N result leaves through the same
// staging tile as whole 128-byte row pieces.  No barrier after the weights are in place, so the loads, arithmetic and
// stores of the wavefronts of a compute unit overlap freely: the bfloat16 kernel is meant to run at the rate of a copy of
// A to C, the float32 one at the rate of its 64-clock products.
// A and C are marked as streams (every byte is touched once); measured, that also leaves the last-level cache to the
// kernel that reads A next.
//
// Serves the forward and the input gradient of the reference's Linear (descriptor `uv,iu,iv` per irrep,
// cuequivariance/group_theory/descriptors/irreps_tp.py:524-547; executed there through FusedTensorProductOp3,
// cuequivariance_torch/primitives/segmented_polynomial_fused_tp.py:40-48).

#include "common.h"
#include "cw_common.h"
#include "u1d_spec.h"
#include "linear_rows_common.h"

namespace cueq {

namespace {

constexpr int kLrStageStride = 144;                 // bytes between the rows of a wavefront's staging tile: 128 of data + 16
constexpr int kLrStageBytes = 32 * kLrStageStride;  // 32 rows

// Number of 16-byte vectors a lane holds for the 32 rows of a unit (rows of K elements of ES bytes).
template <int ES, int KT>
struct LrVectors { static constexpr int n = 32 * KT * ES / 32; };

// The rows of a unit are requested as they lie in memory - every load instruction covers whole 128-byte (or 64-byte) row
// pieces, 8 (16) rows at a time - in passes of at most 128 bytes of k.  Vector i of pass ps: row i * rpi + lane / lpr,
// bytes 128 ps + 16 (lane % lpr), with lpr = 8 lanes per 128-byte piece (4 per 64-byte piece), rpi = 64 / lpr.
// A load that touches a line only in part leaves the rest to a later instruction; marked as a stream, that line would be
// fetched again.
template <int ES, int KT, int NV>
__device__ __forceinline__ void lr_request(uint4 (&xs)[NV], const char* base, int64_t row_bytes, int last_row, int lane) {
  constexpr int RB = 32 * KT * ES;  // bytes of k per row
  static_assert(NV == LrVectors<ES, KT>::n, "one 16-byte vector per lane and kilobyte of the unit");
#pragma unroll
  for (int ps = 0; ps < (RB + 127) / 128; ++ps) {
    const int w = RB - 128 * ps >= 128 ? 128 : 64, lpr = w / 16, rpi = 64 / lpr;
#pragma unroll
    for (int i = 0; i < 32 / rpi; ++i) {
      int r = i * rpi + lane / lpr;
      r = r < last_row ? r : last_row;  // rows past the end repeat the last one
      xs[4 * ps + i] = lr_stream_load(base + r * row_bytes + 128 * ps + 16 * (lane % lpr));
    }
  }
}

// One unit: 32 rows (tile) of one part.  xs holds the rows as requested; they pass through the staging tile to become MFMA
// operands - lane (c, h) takes row c and, of every 64 bytes (2-byte type) or 32 bytes (float) of k, the half h; the weight
// rows in LDS are read the same way, so the order of k inside a row is the same on both sides - and after that `refill()`
// may load xs again.
// FULL: all 32 rows exist (stores without conditions, so that the number of outstanding memory operations at every wait
// is known at compile time and a wait for loads does not also wait for the stores issued after them).
template <typename TI, int KT, int NT, bool FULL, int NV, typename Refill>
__device__ __forceinline__ void lr_unit(uint4 (&xs)[NV], const char* wl, char* stage, TI* crow, int64_t ldc, int rows,
                                        float alpha, int lane, Refill&& refill) {
  constexpr int ES = sizeof(TI);
  constexpr int K = 32 * KT, RB = K * ES;
  constexpr int WRS = RB + 16;
  constexpr int SC = (ES == 2 && NT >= 2) ? 64 : 32;  // result columns staged per pass: 128 bytes (64 for one 2-byte tile)
  constexpr int SRS = kLrStageStride;
  static_assert(NV == LrVectors<ES, KT>::n, "as many operand vectors per lane as requested ones");
  const int c = lane & 31, h = lane >> 5;
  uint4 xf[NV];
#pragma unroll
  for (int ps = 0; ps < (RB + 127) / 128; ++ps) {
    const int w = RB - 128 * ps >= 128 ? 128 : 64, lpr = w / 16, rpi = 64 / lpr;
#pragma unroll
    for (int i = 0; i < 32 / rpi; ++i) *reinterpret_cast<uint4*>(stage + (i * rpi + lane / lpr) * SRS + 16 * (lane % lpr)) = xs[4 * ps + i];
    // 2-byte type: of every 64 bytes the lane half h owns 32 (two vectors); float: of every 32 bytes it owns 16 (one)
#pragma unroll
    for (int j = 0; j < w / 32; ++j)
      xf[4 * ps + j] = *reinterpret_cast<const uint4*>(stage + c * SRS + (ES == 2 ? (j >> 1) * 64 + h * 32 + (j & 1) * 16 : j * 32 + h * 16));
  }
  refill();
  // weight vector v of a row sits where operand vector v of a row of A sat
  auto wvec = [&](int t, int v) -> uint4 {
    const int ps = v >> 2, j = v & 3;
    return *reinterpret_cast<const uint4*>(wl + t * 32 * WRS + 128 * ps + (ES == 2 ? (j >> 1) * 64 + (j & 1) * 16 : j * 32));
  };
  // 2-byte type: the weight fragments of the next 32 result columns are read while the current ones multiply; float:
  // every vector feeds four 64-clock products, which hide the read of the next one
  uint4 af[ES == 2 ? 2 : 1][ES == 2 ? NV : 1];
  if constexpr (ES == 2) {
#pragma unroll
    for (int v = 0; v < NV; ++v) af[0][v] = wvec(0, v);
  }
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    lr_floatx16 acc = lr_floatx16{0};
    if constexpr (ES == 2) {
      if (t + 1 < NT) {
#pragma unroll
        for (int v = 0; v < NV; ++v) af[(t + 1) & 1][v] = wvec(t + 1, v);
      }
#pragma unroll
      for (int v = 0; v < NV; ++v)
        acc = mm_32x32x16<TI>(af[t & 1][v], xf[v], acc);
    } else {
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        const uint4 a = wvec(t, v), b = xf[v];
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), acc, 0, 0, 0);
      }
    }
    // lane (c, h) holds row z = c of the result, columns 32 t + 8 a + 4 h + (0..3)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      if constexpr (ES == 2) {
        const uint2 v = make_uint2(mm_pack<TI>(alpha * acc[4 * a], alpha * acc[4 * a + 1]), mm_pack<TI>(alpha * acc[4 * a + 2], alpha * acc[4 * a + 3]));
        *reinterpret_cast<uint2*>(stage + c * SRS + ((t * 32) % SC + 8 * a + 4 * h) * 2) = v;
      } else {
        *reinterpret_cast<float4*>(stage + c * SRS + (8 * a + 4 * h) * 4) =
            make_float4(alpha * acc[4 * a], alpha * acc[4 * a + 1], alpha * acc[4 * a + 2], alpha * acc[4 * a + 3]);
      }
    }
    if ((t * 32) % SC + 32 == SC || t == NT - 1) {
      const int cols = (t * 32) % SC + 32;  // staged columns of this pass
      const int col0 = t * 32 + 32 - cols;  // first result column of the pass
      const int vpr = cols * ES / 16;       // 16-byte vectors per row
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (j < vpr / 2) {
          const int idx = lane + 64 * j;
          const int r = idx / vpr, cv = idx % vpr;
          if (FULL || r < rows) {
            const uint4 v = *reinterpret_cast<const uint4*>(stage + r * SRS + cv * 16);
            lr_stream_store(v, reinterpret_cast<char*>(crow + static_cast<int64_t>(r) * ldc + col0) + cv * 16);
          }
        }
      }
    }
  }
}

// KT, NT: contraction length and result columns in units of 32.  SETS: operand register sets in rotation (3: the rows of
// unit i + 3 are requested as soon as unit i has taken its operands - for the 2-byte type, whose units are short; 1: the
// next unit's rows are requested into the same registers, and have this unit's products to arrive - float, whose units
// are bound by their 64-clock products).
template <typename TI, int KT, int NT>
__global__ void __launch_bounds__(64 * kLrWaves, 1)
    linear_rows_kernel(const TI* __restrict__ A, int64_t lda, const TI* __restrict__ W, LrParts parts, int nslots, int nparts,
                       int w_contraction_major, TI* __restrict__ C, int64_t ldc, int M, float alpha) {
  constexpr int ES = sizeof(TI);
  constexpr int K = 32 * KT, N = 32 * NT;
  constexpr int WRS = K * ES + 16;  // bytes between weight rows (one row per result column) in LDS
  constexpr int EPV = 16 / ES;
  constexpr int NV = LrVectors<ES, KT>::n;
  extern __shared__ __align__(16) char smem[];
  const int tid = threadIdx.x, lane = tid & 63, c = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  lr_stage_weights<TI, 64 * kLrWaves>(W, parts, nslots, K, N, WRS, w_contraction_major, smem, tid);
  __syncthreads();

  char* stage = smem + nslots * (N * WRS) + wave * kLrStageBytes;
  const char* wlane = smem + c * WRS + h * (ES == 2 ? 32 : 16);
  const int nfull = M / 32;  // tiles of 32 existing rows
  // (slots numbered wavefront-major: when the units do not divide evenly, the wavefronts with one unit more are spread over
  // the CUs and their SIMDs instead of filling the first blocks)
  const int wslot = wave * gridDim.x + blockIdx.x, nw = gridDim.x * kLrWaves;
  // unit = tile * nparts + part; this wavefront takes the units wslot, wslot + nw, ... - walked as (tile, part) pairs
  const int step_t = nw / nparts, step_p = nw % nparts;
  auto advance = [&](int& t, int& p) {
    t += step_t;
    p += step_p;
    if (p >= nparts) { p -= nparts; ++t; }
  };
  auto source = [&](int t, int p) {
    const int tt = t < nfull ? t : nfull - 1;  // past the end: a tile that exists (the values are not used)
    return reinterpret_cast<const char*>(A + static_cast<int64_t>(tt) * 32 * lda + parts.part[p].a_off);
  };
  const int64_t row_bytes = lda * ES;
  const int64_t total_full = static_cast<int64_t>(nfull) * nparts;
  if (wslot < total_full) {
    const int mine = static_cast<int>((total_full - wslot + nw - 1) / nw);  // units of this wavefront
    int t = wslot / nparts, p = wslot % nparts;  // the unit worked on
    int rt = t, rp = p;                          // the unit requested
#define LR_PHASE(XS, AFTER)                                                                                                                  \
    {                                                                                                                                         \
      const char* src = source(rt, rp);                                                                                                       \
      lr_unit<TI, KT, NT, true>(XS, wlane + parts.part[p].slot * (N * WRS), stage, C + static_cast<int64_t>(t) * 32 * ldc + parts.part[p].c_off, \
                                ldc, 32, alpha, lane, AFTER);                                                                                 \
      advance(rt, rp);                                                                                                                        \
      advance(t, p);                                                                                                                          \
    }
#define LR_NEXT(XS) [&]() { lr_request<ES, KT>(XS, src, row_bytes, 31, lane); __builtin_amdgcn_sched_barrier(0); }
    if constexpr (ES == 2) {
      // Three operand sets in rotation: the rows of unit i + 3 are requested as soon as unit i has taken its operands.
      // The loop body is three units without a branch in between (one basic block: the requests stay where they are
      // written); the one or two units left over follow it.
      uint4 x0[NV], x1[NV], x2[NV];
      lr_request<ES, KT>(x0, source(rt, rp), row_bytes, 31, lane);
      advance(rt, rp);
      lr_request<ES, KT>(x1, source(rt, rp), row_bytes, 31, lane);
      advance(rt, rp);
      lr_request<ES, KT>(x2, source(rt, rp), row_bytes, 31, lane);
      advance(rt, rp);
      for (int it = 0; it < mine / 3; ++it) {
        LR_PHASE(x0, LR_NEXT(x0))
        LR_PHASE(x1, LR_NEXT(x1))
        LR_PHASE(x2, LR_NEXT(x2))
      }
      if (mine % 3 >= 1) LR_PHASE(x0, [&]() { (void)src; })
      if (mine % 3 == 2) LR_PHASE(x1, [&]() { (void)src; })
    } else {
      // float: one operand set; the next unit's rows are requested right after this unit's operands left it and have
      // the whole of its products (64 clocks each) to arrive
      uint4 x0[NV];
      lr_request<ES, KT>(x0, source(rt, rp), row_bytes, 31, lane);
      advance(rt, rp);
      for (int it = 0; it < mine; ++it) LR_PHASE(x0, LR_NEXT(x0))
    }
#undef LR_NEXT
#undef LR_PHASE
  }
  if (M % 32 != 0) {  // the units of the last, partial tile
    for (int p = wslot; p < nparts; p += nw) {
      uint4 xs[NV];
      lr_request<ES, KT>(xs, reinterpret_cast<const char*>(A + static_cast<int64_t>(nfull) * 32 * lda + parts.part[p].a_off), row_bytes, M - nfull * 32 - 1, lane);
      lr_unit<TI, KT, NT, false>(xs, wlane + parts.part[p].slot * (N * WRS), stage, C + static_cast<int64_t>(nfull) * 32 * ldc + parts.part[p].c_off, ldc,
                                 M - nfull * 32, alpha, lane, []() {});
    }
  }
}

}  // namespace

}  // namespace cueq

// table: host memory, nparts rows of (a_off, w_off, c_off) in elements
extern "C" int cueq_linear_rows(int32_t dtype, int32_t w_contraction_major, int64_t M, int64_t N, int64_t K, const void* A, int64_t lda,
                                const void* W, int64_t w_numel, void* C, int64_t ldc, const int64_t* table, int64_t nparts, double alpha, void* stream_) {
  using namespace cueq;
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(dtype == CUEQ_BF16 || dtype == CUEQ_F16 || dtype == CUEQ_F32, CUEQ_ERR_UNSUPPORTED, "linear_rows: bfloat16, half or float32");
  CUEQ_REQUIRE(M >= 0 && N > 0 && K > 0 && nparts >= 0, CUEQ_ERR_INVALID, "linear_rows: bad extents");
  CUEQ_REQUIRE(N % 32 == 0 && K % 32 == 0 && N <= 128 && K <= 128, CUEQ_ERR_UNSUPPORTED, "linear_rows: K and N must be 32, 64, 96 or 128");
  CUEQ_REQUIRE(nparts <= kLrMaxParts, CUEQ_ERR_TOO_LARGE, "linear_rows: at most %d parts per launch", kLrMaxParts);
  if (M == 0 || nparts == 0) return CUEQ_OK;
  CUEQ_REQUIRE(A && W && C && table, CUEQ_ERR_INVALID, "linear_rows: null operand");
  CUEQ_REQUIRE(M <= (1ll << 31) - 64, CUEQ_ERR_TOO_LARGE, "linear_rows: too many rows");
  const int es = dtype == CUEQ_F32 ? 4 : 2, epv = 16 / es;
  CUEQ_REQUIRE(lda % epv == 0 && ldc % epv == 0 && reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(C) % 16 == 0,
               CUEQ_ERR_UNSUPPORTED, "linear_rows: row strides and pointers must be multiples of 16 bytes");
  LrParts parts;
  int nslots = 0;
  for (int64_t p = 0; p < nparts; ++p) {
    const int64_t a_off = table[3 * p], w_off = table[3 * p + 1], c_off = table[3 * p + 2];
    CUEQ_REQUIRE(a_off >= 0 && a_off + K <= lda && c_off >= 0 && c_off + N <= ldc && w_off >= 0 && w_off + K * N <= w_numel && a_off % epv == 0 &&
                     c_off % epv == 0 && w_off % epv == 0,
                 CUEQ_ERR_INVALID, "linear_rows: part %lld: offsets must lie inside a row / the weights and be multiples of 16 bytes",
                 static_cast<long long>(p));
    int s = 0;
    while (s < nslots && parts.w_off[s] != w_off) ++s;
    if (s == nslots) {
      CUEQ_REQUIRE(nslots < kLrMaxSlots, CUEQ_ERR_TOO_LARGE, "linear_rows: at most %d distinct weight blocks per launch", kLrMaxSlots);
      parts.w_off[nslots++] = w_off;
    }
    parts.part[p] = LrPart{static_cast<int32_t>(a_off), static_cast<int32_t>(c_off), s};
  }
  const size_t lds = static_cast<size_t>(nslots) * N * (es * K + 16) + static_cast<size_t>(kLrWaves) * kLrStageBytes;
  CUEQ_REQUIRE(lds <= 160 * 1024, CUEQ_ERR_TOO_LARGE, "linear_rows: the weight blocks of one launch do not fit the local data share");
  const int64_t total = ((M + 31) / 32) * nparts;
  int64_t gx = (total + kLrWaves - 1) / kLrWaves;
  if (gx > device_cus()) gx = device_cus();
  KernelTimer timer("linear_rows", stream);
#define LR(TI_, KT_, NT_)                                                                                                                     \
  do {                                                                                                                                        \
    auto kfn = linear_rows_kernel<TI_, KT_, NT_>;                                                                                             \
    CUEQ_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kfn), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds))); \
    hipLaunchKernelGGL(kfn, dim3(static_cast<unsigned>(gx)), dim3(64 * kLrWaves), lds, stream, static_cast<const TI_*>(A), lda,               \
                       static_cast<const TI_*>(W), parts, nslots, static_cast<int>(nparts), w_contraction_major, static_cast<TI_*>(C), ldc,   \
                       static_cast<int>(M), static_cast<float>(alpha));                                                                       \
  } while (0)
#define LR_N(TI_, KT_)                                                                                                                         \
  switch (N / 32) { case 1: LR(TI_, KT_, 1); break; case 2: LR(TI_, KT_, 2); break; case 3: LR(TI_, KT_, 3); break; default: LR(TI_, KT_, 4); break; }
#define LR_K(TI_)                  \
  switch (K / 32) {                \
    case 1: LR_N(TI_, 1); break;   \
    case 2: LR_N(TI_, 2); break;   \
    case 3: LR_N(TI_, 3); break;   \
    default: LR_N(TI_, 4); break;  \
  }
  if (dtype == CUEQ_F32) { LR_K(float) } else if (dtype == CUEQ_F16) { LR_K(f16bits) } else { LR_K(uint16_t) }
#undef LR_K
#undef LR_N
#undef LR
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}
