// Weight gradient of Linear-like operations on rows that keep the irrep component contiguous (`mul_ir`: element
// (channel u, component i) of a block of D components at u * D + i), bfloat16 or float32 elements, float32 accumulation:
//   dW_p[u, v] = alpha * sum_z sum_{i < D_p} A[z, a_p + u * D_p + i] * G[z, c_p + v * D_p + i]      (K x N per part p)
// as partial sums over row chunks that the caller adds in order (no atomics, bit-reproducible).  The reference reaches this
// product through autograd of its dense kernel after transposing the rows to channel-contiguous ones
// (cuequivariance_torch/primitives/transpose.py:83-183, operations/linear.py:153-191); here the rows are read as they lie.
//
// A block of 256 threads owns one (part, chunk of rows).  Per step it takes 16 rows (8 of float): the rows are loaded as
// they lie (whole 128-byte lines per instruction) and every element is scattered into LDS planes
// [component][row half][channel][8 (4) rows = 16 bytes] - the slot addresses are D registers per operand plus immediate
// offsets - from which the lanes read MFMA operands with the rows as contraction index: one 16-byte read per 32 x 32 tile
// side, component and step, 512 contiguous bytes per half wavefront.  The four wavefronts split
// the K x N result two by two.  Parts of different D run in one launch (the block branches once on its part's D), with
// chunk counts in proportion to D + 1 so that all blocks carry about the same work.

#include "common.h"
#include "cw_common.h"
#include "u1d_spec.h"

namespace cueq {

namespace {

typedef float dw_floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 dw_bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kDwMaxParts = 32;

struct DwParts {
  int32_t a_off[kDwMaxParts], c_off[kDwMaxParts], d[kDwMaxParts];
  int32_t first[kDwMaxParts + 1];  // first item (row of the partial buffer) of a part; items of a part are its chunks
};

template <typename TI, int D>
__device__ __forceinline__ void dw_body(const TI* __restrict__ A, int64_t lda, const TI* __restrict__ G, int64_t ldg, float* __restrict__ P,
                                        int K, int N, int64_t z_begin, int64_t z_end, float alpha, char* smem) {
  constexpr int ES = sizeof(TI);
  constexpr int EPV = 16 / ES;    // elements per 16-byte vector
  constexpr int ZR = 2 * EPV;     // rows per step: 16 (2-byte type) or 8 (float)
  constexpr int ZH = ZR / 2;      // rows per 16-byte slot
  constexpr int EPL = 128 / ES;   // elements per 128-byte line
  const int tid = threadIdx.x, lane = tid & 63, c = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int KT = K / 32, NT = N / 32;
  const int TU = (KT + 1) / 2, TV = (NT + 1) / 2;  // tiles of a wavefront along u and v (at most 2 x 2)
  // planes [component][row half][channel][16 bytes = ZH rows]; 16 bytes more per plane so that planes start on different banks
  const int PLX = K * 32 + 16, PLG = N * 32 + 16;
  char* sx = smem;
  char* sg = smem + D * PLX;

  // Loads: eight lanes per 128-byte line; instruction v of a thread takes line v * (32 / ZR) + gidx / ZR of row gidx % ZR
  // (gidx = tid / 8), so every instruction covers whole lines and the row of a thread is the same for all v.
  // Element j of that vector is element E = E0 + 128 v + j of the row piece, E0 = (gidx / ZR) * EPL + (tid % 8) * EPV, i.e.
  // channel E / D, component E % D.  With r0 = E0 % D the slot of element (v, j) is  slot[(128 v + j) % D] + 16 * ((128 v + j) / D),
  // where slot[k] is the address of (channel E0 / D + (r0 + k) / D, component (r0 + k) % D, the thread's row): D address
  // registers per operand, everything else is an immediate offset.
  const int gidx = tid >> 3, l8 = tid & 7;
  const int row = gidx % ZR, line0 = gidx / ZR;
  const int E0 = line0 * EPL + l8 * EPV, r0 = E0 % D, u0 = E0 / D;
  const int VRX = K * D / EPV, VRG = N * D / EPV;  // 16-byte vectors per row piece
  const TI* xp = A + row * lda + E0;
  const TI* gp = G + row * ldg + E0;
  char* xslot[D];
  char* gslot[D];
#pragma unroll
  for (int k = 0; k < D; ++k) {
    const int du = (r0 + k) / D, i = (r0 + k) % D;
    xslot[k] = sx + i * PLX + (row / ZH) * (K * 16) + (u0 + du) * 16 + (row % ZH) * ES;
    gslot[k] = sg + i * PLG + (row / ZH) * (N * 16) + (u0 + du) * 16 + (row % ZH) * ES;
  }

  uint4 rx[D], rg[D];
  auto load_step = [&](int64_t z) {
    const bool ok = z + row < z_end;
#pragma unroll
    for (int v = 0; v < D; ++v) {
      const int vi = (v * (32 / ZR) + line0) * 8 + l8;  // the vector's place in the row piece
      rx[v] = (ok && vi < VRX) ? *reinterpret_cast<const uint4*>(xp + z * lda + v * (32 / ZR) * EPL) : make_uint4(0, 0, 0, 0);
      rg[v] = (ok && vi < VRG) ? *reinterpret_cast<const uint4*>(gp + z * ldg + v * (32 / ZR) * EPL) : make_uint4(0, 0, 0, 0);
    }
  };
  auto scatter = [&](const uint4 (&r)[D], char* const (&slot)[D], int VR) {
#pragma unroll
    for (int v = 0; v < D; ++v) {
      if ((v * (32 / ZR) + line0) * 8 + l8 >= VR) continue;
      const uint32_t w[4] = {r[v].x, r[v].y, r[v].z, r[v].w};
#pragma unroll
      for (int j = 0; j < EPV; ++j) {
        const int sidx = 128 * v + j;
        char* dst = slot[sidx % D] + 16 * (sidx / D);
        if constexpr (ES == 2) *reinterpret_cast<uint16_t*>(dst) = static_cast<uint16_t>(w[j >> 1] >> (16 * (j & 1)));
        else *reinterpret_cast<uint32_t*>(dst) = w[j];
      }
    }
  };

  dw_floatx16 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b) acc[a][b] = dw_floatx16{0};

  if (z_begin < z_end) load_step(z_begin);
  for (int64_t z = z_begin; z < z_end; z += ZR) {
    __syncthreads();  // the previous step's reads are done
    scatter(rx, xslot, VRX);
    scatter(rg, gslot, VRG);
    __syncthreads();
    if (z + ZR < z_end) load_step(z + ZR);
#pragma unroll
    for (int i = 0; i < D; ++i) {
      uint4 fa[2], fb[2];
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        const int tu = wm * TU + a;
        if (a < TU && tu < KT) fa[a] = *reinterpret_cast<const uint4*>(sx + i * PLX + h * (K * 16) + (32 * tu + c) * 16);
        const int tv = wn * TV + a;
        if (a < TV && tv < NT) fb[a] = *reinterpret_cast<const uint4*>(sg + i * PLG + h * (N * 16) + (32 * tv + c) * 16);
      }
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          if (!(a < TU && wm * TU + a < KT && b < TV && wn * TV + b < NT)) continue;
          if constexpr (ES == 2) {
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(dw_bf16x8, fa[a]), __builtin_bit_cast(dw_bf16x8, fb[b]), acc[a][b], 0, 0, 0);
          } else {
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(fa[a].x), __uint_as_float(fb[b].x), acc[a][b], 0, 0, 0);
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(fa[a].y), __uint_as_float(fb[b].y), acc[a][b], 0, 0, 0);
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(fa[a].z), __uint_as_float(fb[b].z), acc[a][b], 0, 0, 0);
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(fa[a].w), __uint_as_float(fb[b].w), acc[a][b], 0, 0, 0);
          }
        }
    }
  }
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int tu = wm * TU + a, tv = wn * TV + b;
      if (!(a < TU && tu < KT && b < TV && tv < NT)) continue;
      const int col = 32 * tv + c;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = 32 * tu + 8 * (r >> 2) + 4 * h + (r & 3);
        P[static_cast<int64_t>(row) * N + col] = alpha * acc[a][b][r];
      }
    }
}

template <typename TI>
__global__ void __launch_bounds__(256) linear_dw_mul_ir_kernel(const TI* __restrict__ A, int64_t lda, const TI* __restrict__ G, int64_t ldg,
                                                               DwParts parts, int nparts, float* __restrict__ P, int K, int N, int64_t rows,
                                                               float alpha) {
  extern __shared__ __align__(16) char smem[];
  const int item = blockIdx.x;
  int p = 0;
  while (p + 1 < nparts && parts.first[p + 1] <= item) ++p;
  const int chunk = item - parts.first[p], chunks = parts.first[p + 1] - parts.first[p];
  constexpr int ZR = 32 / sizeof(TI);
  const int64_t rpc = (((rows + chunks - 1) / chunks + ZR - 1) / ZR) * ZR;  // rows per chunk: whole steps
  const int64_t z_begin = chunk * rpc;
  int64_t z_end = z_begin + rpc;
  if (z_end > rows) z_end = rows;
  const TI* a = A + parts.a_off[p];
  const TI* g = G + parts.c_off[p];
  float* out = P + static_cast<int64_t>(item) * K * N;
  switch (parts.d[p]) {
    case 1: dw_body<TI, 1>(a, lda, g, ldg, out, K, N, z_begin, z_end, alpha, smem); break;
    case 3: dw_body<TI, 3>(a, lda, g, ldg, out, K, N, z_begin, z_end, alpha, smem); break;
    case 5: dw_body<TI, 5>(a, lda, g, ldg, out, K, N, z_begin, z_end, alpha, smem); break;
    default: dw_body<TI, 7>(a, lda, g, ldg, out, K, N, z_begin, z_end, alpha, smem); break;
  }
}

// chunk counts per part, in proportion to D + 1 (measured: a step costs about as much again as one of its D components),
// about two blocks per compute unit in all; every chunk at least 64 rows
int64_t dw_plan(int64_t rows, const int64_t* table, int nparts, int32_t* first) {
  int64_t dsum = 0;
  for (int p = 0; p < nparts; ++p) dsum += table[3 * p + 2] + 1;
  const int64_t budget = static_cast<int64_t>(device_cus()) * 2;
  const int64_t most = (rows + 63) / 64 > 0 ? (rows + 63) / 64 : 1;
  int64_t total = 0;
  for (int p = 0; p < nparts; ++p) {
    int64_t n = budget * (table[3 * p + 2] + 1) / (dsum > 0 ? dsum : 1);
    if (n > most) n = most;
    if (n < 1) n = 1;
    first[p] = static_cast<int32_t>(total);
    total += n;
  }
  first[nparts] = static_cast<int32_t>(total);
  return total;
}

}  // namespace

}  // namespace cueq

// table: host memory, nparts rows of (a_off, c_off, D).  first_item (nparts + 1 entries, may be null) receives the first row
// of every part in the partial buffer; returns the number of rows (K * N floats each) that buffer needs.
extern "C" int64_t cueq_linear_dw_mul_ir_items(int64_t rows, const int64_t* table, int32_t nparts, int32_t* first_item) {
  using namespace cueq;
  if (!table || nparts < 1 || nparts > kDwMaxParts) return -1;
  int32_t first[kDwMaxParts + 1];
  const int64_t total = dw_plan(rows, table, nparts, first);
  if (first_item)
    for (int p = 0; p <= nparts; ++p) first_item[p] = first[p];
  return total;
}

extern "C" int cueq_linear_dw_mul_ir(int32_t dtype, int64_t K, int64_t N, int64_t rows, const void* A, int64_t lda, const void* G, int64_t ldg,
                                     const int64_t* table, int32_t nparts, float* partials, double alpha, void* stream_) {
  using namespace cueq;
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(dtype == CUEQ_BF16 || dtype == CUEQ_F32, CUEQ_ERR_UNSUPPORTED, "linear_dw_mul_ir: bfloat16 or float32");
  CUEQ_REQUIRE(rows >= 0 && nparts >= 1 && nparts <= kDwMaxParts, CUEQ_ERR_INVALID, "linear_dw_mul_ir: 1 to %d parts", kDwMaxParts);
  CUEQ_REQUIRE(K > 0 && N > 0 && K % 32 == 0 && N % 32 == 0 && K <= 128 && N <= 128, CUEQ_ERR_UNSUPPORTED,
               "linear_dw_mul_ir: K and N must be 32, 64, 96 or 128");
  CUEQ_REQUIRE(A && G && partials && table, CUEQ_ERR_INVALID, "linear_dw_mul_ir: null operand");
  const int es = dtype == CUEQ_F32 ? 4 : 2, epv = 16 / es;
  CUEQ_REQUIRE(lda % epv == 0 && ldg % epv == 0 && reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(G) % 16 == 0,
               CUEQ_ERR_UNSUPPORTED, "linear_dw_mul_ir: row strides and pointers must be multiples of 16 bytes");
  DwParts parts;
  int dmax = 1;
  for (int p = 0; p < nparts; ++p) {
    const int64_t a_off = table[3 * p], c_off = table[3 * p + 1], d = table[3 * p + 2];
    CUEQ_REQUIRE(d == 1 || d == 3 || d == 5 || d == 7, CUEQ_ERR_UNSUPPORTED, "linear_dw_mul_ir: blocks of 1, 3, 5 or 7 components");
    CUEQ_REQUIRE(a_off >= 0 && a_off + K * d <= lda && c_off >= 0 && c_off + N * d <= ldg && a_off % epv == 0 && c_off % epv == 0, CUEQ_ERR_INVALID,
                 "linear_dw_mul_ir: part %d: offsets must lie inside a row and be multiples of 16 bytes", p);
    parts.a_off[p] = static_cast<int32_t>(a_off);
    parts.c_off[p] = static_cast<int32_t>(c_off);
    parts.d[p] = static_cast<int32_t>(d);
    if (d > dmax) dmax = static_cast<int>(d);
  }
  const int64_t items = dw_plan(rows, table, nparts, parts.first);
  const size_t lds = static_cast<size_t>(dmax) * ((K + N) * 32 + 32);
  CUEQ_REQUIRE(lds <= 160 * 1024, CUEQ_ERR_TOO_LARGE, "linear_dw_mul_ir: the planes do not fit the local data share");
  KernelTimer timer("linear_dw_mul_ir", stream);
#define DW(TI_)                                                                                                                               \
  do {                                                                                                                                        \
    auto kfn = linear_dw_mul_ir_kernel<TI_>;                                                                                                  \
    CUEQ_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kfn), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds))); \
    hipLaunchKernelGGL(kfn, dim3(static_cast<unsigned>(items)), dim3(256), lds, stream, static_cast<const TI_*>(A), lda, static_cast<const TI_*>(G), \
                       ldg, parts, nparts, partials, static_cast<int>(K), static_cast<int>(N), rows, static_cast<float>(alpha));              \
  } while (0)
  if (dtype == CUEQ_F32) DW(float); else DW(uint16_t);
#undef DW
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}
