// Weight gradient of Linear-like operations on rows that keep the irrep component contiguous (`mul_ir`: element
// (channel u, component i) of a block of D components at u * D + i), bfloat16 or float32 elements, float32 accumulation:
//   dW_p[u, v] = alpha * sum_z sum_{i < D_p} A[z, a_p + u * D_p + i] * G[z, c_p + v * D_p + i]      (K x N per part p)
// as partial sums over row chunks that the caller adds in order (no atomics, bit-reproducible).  The reference reaches this
// product through autograd of its dense kernel after transposing the rows to channel-contiguous ones
// (cuequivariance_torch/primitives/transpose.py:83-183, operations/linear.py:153-191); here the rows are read as they lie.
//
// A block of 256 threads owns one (part, chunk of rows).  Per step it takes 16 rows (8 of float): the rows are loaded as
// they lie (whole 128-byte lines per instruction) and every element is scattered into LDS planes
// [component][row half][channel][8 (4) rows = 16 bytes] - two rows per store after an exchange between neighbouring
// lanes, the slot addresses being D registers per operand plus immediate offsets - from which the lanes read MFMA operands with the rows as contraction index: one 16-byte read per 32 x 32 tile
// side, component and step, 512 contiguous bytes per half wavefront.  The four wavefronts split
// the K x N result two by two.  Parts of different D run in one launch (the block branches once on its part's D), with
// chunk counts in proportion to D + 1/2 so that all blocks carry about the same work.

#include "common.h"
#include "cw_common.h"
#include "u1d_spec.h"

#include <type_traits>

namespace cueq {

namespace {

typedef float dw_floatx16 __attribute__((ext_vector_type(16)));

constexpr int kDwMaxParts = 32;
// Blocks of up to this many components request their rows two steps ahead (two register sets); with five components the
// second set spills and one set measured faster (bfloat16, 200 000 rows: 95 against 112 microseconds).
#ifndef DW_TWO_SETS_UP_TO
#define DW_TWO_SETS_UP_TO 3
#endif

struct DwParts {
  int32_t a_off[kDwMaxParts], c_off[kDwMaxParts], d[kDwMaxParts];
  int32_t first[kDwMaxParts + 1];  // first item (row of the partial buffer) of a part; items of a part are its chunks
};

typedef uint32_t dw_u32x4 __attribute__((ext_vector_type(4)));
// 16-byte load marked as a stream: every byte of A and G is read once
template <typename T>
__device__ __forceinline__ uint4 dw_stream_load(const T* p) {
  const dw_u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const dw_u32x4*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}

// Block-wide barrier that waits for the wavefront's LDS operations only.  __syncthreads() also waits for every outstanding
// global load, which would end the requests made two steps ahead at each of the two barriers of a step.
__device__ __forceinline__ void dw_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

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
  const int KT = K / 32, NT = N / 32;
  // The four wavefronts split the KT x NT tiles of 32 x 32 as a grid gu x gv, TU x TV tiles each (at most 2 x 2): 4 x 1 or
  // 1 x 4 when one side is a single tile, else 2 x 2.  A tile index past the end is clamped (computed again, not stored).
  const int gu = NT == 1 ? 4 : (KT == 1 ? 1 : 2), gv = 4 / gu;
  const int wm = wave / gv, wn = wave % gv;
  const int TU = (KT + gu - 1) / gu, TV = (NT + gv - 1) / gv;
  // planes [component][row half][channel][16 bytes = ZH rows]; 16 bytes more per plane so that planes start on different banks
  const int PLX = K * 32 + 16, PLG = N * 32 + 16;
  char* sx = smem;
  char* sg = smem + D * PLX;

  // Loads: eight lanes per 128-byte line; instruction v of a thread takes line v * (32 / ZR) + gidx / ZR of row gidx % ZR
  // (gidx = tid / 8), so every instruction covers whole lines and the row of a thread is the same for all v.
  // Element j of that vector is element E = E0 + 128 v + j of the row piece, E0 = (gidx / ZR) * EPL + (tid % 8) * EPV, i.e.
  // channel E / D, component E % D.
  // Stores into the planes: rows z and z + 1 of one (channel, component) are neighbours in a slot and sit in lanes 8 apart,
  // so the two lanes exchange their vectors (one DPP move per register) and each writes half of the elements for both
  // rows: the lane of the even row the elements j = 2 m (2-byte type: 4-byte writes) or j = 0, 1 (float: 8-byte writes),
  // the lane of the odd row the others - half the LDS instructions of element-wise stores.  With F0 = E0 + the lane's
  // first element and r0 = F0 % D, the slot of its write number m of vector v is  slot[q % D] + 16 * (q / D),
  // q = 128 v + step * m, where slot[k] is the address of (channel F0 / D + (r0 + k) / D, component (r0 + k) % D, the row
  // pair): D address registers per operand, everything else is an immediate offset.
  const int gidx = tid >> 3, l8 = tid & 7;
  const int row = gidx % ZR, line0 = gidx / ZR, odd = row & 1;
  const int E0 = line0 * EPL + l8 * EPV;
  const int F0 = E0 + (ES == 2 ? odd : 2 * odd), r0 = F0 % D, u0 = F0 / D;
  const int VRX = K * D / EPV, VRG = N * D / EPV;  // 16-byte vectors per row piece
  char* xslot[D];
  char* gslot[D];
#pragma unroll
  for (int k = 0; k < D; ++k) {
    const int du = (r0 + k) / D, i = (r0 + k) % D;
    xslot[k] = sx + i * PLX + (row / ZH) * (K * 16) + (u0 + du) * 16 + ((row % ZH) & ~1) * ES;
    gslot[k] = sg + i * PLG + (row / ZH) * (N * 16) + (u0 + du) * 16 + ((row % ZH) & ~1) * ES;
  }
  // 2-byte type: bytes of {partner (4-7), own (0-3)} that make (row z, row z + 1) of the lane's element of a register
  const uint32_t pair_sel = odd ? 0x03020706u : 0x05040100u;

  // two register sets: the rows two steps ahead are requested while the current step multiplies.  The requests carry no
  // condition (a row past the end of the chunk repeats the last one, a vector past the row piece repeats the first): after a
  // conditional load the compiler waits for all outstanding loads at once.  What must not count is zeroed when it is stored.
  constexpr int SETS = D <= DW_TWO_SETS_UP_TO ? 2 : 1;
  uint4 rx[SETS][D], rg[SETS][D];
  bool live[SETS];
  // (a vector past the row piece - extents below 128 only - repeats the lane's last one that exists)
  const int xlim = VRX - 1 - line0 * 8 - l8 >= 0 ? ((VRX - 1 - line0 * 8 - l8) / (8 * (32 / ZR))) * (32 / ZR) * EPL : 0;
  const int glim = VRG - 1 - line0 * 8 - l8 >= 0 ? ((VRG - 1 - line0 * 8 - l8) / (8 * (32 / ZR))) * (32 / ZR) * EPL : 0;
  // (a lane whose first vector lies past the row piece - pieces shorter than 128 elements - requests the piece's first
  // vector instead: nothing is read outside the piece, which for the last row of a tensor would be outside the tensor)
  const TI* xp = A + (line0 * 8 + l8 < VRX ? E0 : 0);
  const TI* gp = G + (line0 * 8 + l8 < VRG ? E0 : 0);
  auto load_step = [&](uint4 (&qx)[D], uint4 (&qg)[D], bool& ok, int64_t z) {
    ok = z + row < z_end;
    const int64_t zz = ok ? z + row : z_end - 1;
#pragma unroll
    for (int v = 0; v < D; ++v) {
      qx[v] = dw_stream_load(xp + zz * lda + min(v * (32 / ZR) * EPL, xlim));
      qg[v] = dw_stream_load(gp + zz * ldg + min(v * (32 / ZR) * EPL, glim));
    }
  };
  auto scatter = [&](const uint4 (&r)[D], char* const (&slot)[D], int VR, bool ok) {
#pragma unroll
    for (int v = 0; v < D; ++v) {
      const uint32_t w[4] = {ok ? r[v].x : 0u, ok ? r[v].y : 0u, ok ? r[v].z : 0u, ok ? r[v].w : 0u};
      uint32_t pw[4];  // the same vector of the neighbouring row (lane ^ 8: rotation by 8 inside a row of 16 lanes)
#pragma unroll
      for (int m = 0; m < 4; ++m) pw[m] = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(w[m]), 0x128, 0xf, 0xf, true));
      if ((v * (32 / ZR) + line0) * 8 + l8 >= VR) continue;
      if constexpr (ES == 2) {
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          const int q = 128 * v + 2 * m;
          *reinterpret_cast<uint32_t*>(slot[q % D] + 16 * (q / D)) = __builtin_amdgcn_perm(pw[m], w[m], pair_sel);
        }
      } else {
#pragma unroll
        for (int m = 0; m < 2; ++m) {
          const int q = 128 * v + m;
          const uint32_t mine = odd ? w[2 + m] : w[m], other = odd ? pw[2 + m] : pw[m];
          *reinterpret_cast<uint2*>(slot[q % D] + 16 * (q / D)) = odd ? make_uint2(other, mine) : make_uint2(mine, other);
        }
      }
    }
  };

  dw_floatx16 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b) acc[a][b] = dw_floatx16{0};

  // tile offsets of the wavefront inside a plane (clamped) and whether the tile exists
  int xo[2], go[2];
  bool xv[2], gv_ok[2];
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    const int tu = wm * TU + a, tv = wn * TV + a;
    xv[a] = a < TU && tu < KT;
    gv_ok[a] = a < TV && tv < NT;
    xo[a] = h * (K * 16) + (32 * (xv[a] ? tu : 0) + c) * 16;
    go[a] = h * (N * 16) + (32 * (gv_ok[a] ? tv : 0) + c) * 16;
  }
  // TA x TB tiles per wavefront as compile-time numbers: no branch inside a step
  auto run = [&](auto ta_, auto tb_) {
    constexpr int TA = decltype(ta_)::value, TB = decltype(tb_)::value;
    auto products = [&]() {
#pragma unroll
      for (int i = 0; i < D; ++i) {
        uint4 fa[TA], fb[TB];
#pragma unroll
        for (int a = 0; a < TA; ++a) fa[a] = *reinterpret_cast<const uint4*>(sx + i * PLX + xo[a]);
#pragma unroll
        for (int b = 0; b < TB; ++b) fb[b] = *reinterpret_cast<const uint4*>(sg + i * PLG + go[b]);
#pragma unroll
        for (int a = 0; a < TA; ++a)
#pragma unroll
          for (int b = 0; b < TB; ++b) {
            if constexpr (ES == 2) {
              acc[a][b] = mm_32x32x16<TI>(fa[a], fb[b], acc[a][b]);
            } else {
              acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(fa[a].x), __uint_as_float(fb[b].x), acc[a][b], 0, 0, 0);
              acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(fa[a].y), __uint_as_float(fb[b].y), acc[a][b], 0, 0, 0);
              acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(fa[a].z), __uint_as_float(fb[b].z), acc[a][b], 0, 0, 0);
              acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(fa[a].w), __uint_as_float(fb[b].w), acc[a][b], 0, 0, 0);
            }
          }
        if (i % 2 == 1) __builtin_amdgcn_sched_barrier(0);  // (operands of at most two components in registers at a time)
      }
    };
    const int64_t nsteps = (z_end - z_begin + ZR - 1) / ZR;
    int64_t z = z_begin;
#define DW_STEP(k_)                                          \
    {                                                        \
      dw_lds_barrier(); /* the previous step's reads are done */ \
      scatter(rx[k_], xslot, VRX, live[k_]);                 \
      scatter(rg[k_], gslot, VRG, live[k_]);                 \
      dw_lds_barrier();                                      \
      load_step(rx[k_], rg[k_], live[k_], z + SETS * ZR);    \
      products();                                            \
      z += ZR;                                               \
    }
    if constexpr (SETS == 2) {
      for (int64_t it = 0; it < nsteps / 2; ++it) {
        DW_STEP(0)
        DW_STEP(1)
      }
      if (nsteps & 1) DW_STEP(0)
    } else {
      for (int64_t it = 0; it < nsteps; ++it) DW_STEP(0)
    }
#undef DW_STEP
  };
  if (z_begin >= z_end) z_end = z_begin;  // (an empty chunk: nothing is loaded, zeros are written)
  if (z_begin < z_end) {
    load_step(rx[0], rg[0], live[0], z_begin);
    if constexpr (SETS == 2) load_step(rx[SETS - 1], rg[SETS - 1], live[SETS - 1], z_begin + ZR);
    using one = std::integral_constant<int, 1>;
    using two = std::integral_constant<int, 2>;
    if (TU == 2 && TV == 2) run(two{}, two{});
    else if (TU == 2) run(two{}, one{});
    else if (TV == 2) run(one{}, two{});
    else run(one{}, one{});
  }
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      if (!(xv[a] && gv_ok[b])) continue;
      const int col = 32 * (wn * TV + b) + c;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = 32 * (wm * TU + a) + 8 * (r >> 2) + 4 * h + (r & 3);
        P[static_cast<int64_t>(row) * N + col] = alpha * acc[a][b][r];
      }
    }
}

// DMAX: the largest D among the parts of the launch (the registers of the kernel are those of its largest body).  Two blocks
// per compute unit (three measured slower: the blocks share the LDS pipeline).
template <typename TI, int DMAX>
__global__ void __launch_bounds__(256, 2) linear_dw_mul_ir_kernel(const TI* __restrict__ A, int64_t lda, const TI* __restrict__ G,
                                                                                   int64_t ldg, DwParts parts, int nparts, float* __restrict__ P,
                                                                                   int K, int N, int64_t rows, float alpha) {
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
  const int d = parts.d[p];
  if (d == 1) dw_body<TI, 1>(a, lda, g, ldg, out, K, N, z_begin, z_end, alpha, smem);
  if constexpr (DMAX >= 3) { if (d == 3) dw_body<TI, 3>(a, lda, g, ldg, out, K, N, z_begin, z_end, alpha, smem); }
  if constexpr (DMAX >= 5) { if (d == 5) dw_body<TI, 5>(a, lda, g, ldg, out, K, N, z_begin, z_end, alpha, smem); }
  if constexpr (DMAX >= 7) { if (d == 7) dw_body<TI, 7>(a, lda, g, ldg, out, K, N, z_begin, z_end, alpha, smem); }
}

// chunk counts per part, in proportion to D + 1/2 (measured: a step costs about half as much again as one of its D
// components), as many blocks in all as are resident at one time; every chunk at least 64 rows
int64_t dw_plan(int64_t rows, const int64_t* table, int nparts, int32_t* first) {
  int64_t dsum = 0;
  for (int p = 0; p < nparts; ++p) dsum += 2 * table[3 * p + 2] + 1;
  const int64_t budget = static_cast<int64_t>(device_cus()) * 2;  // what is resident at one time
  const int64_t most = (rows + 63) / 64 > 0 ? (rows + 63) / 64 : 1;
  int64_t total = 0;
  for (int p = 0; p < nparts; ++p) {
    int64_t n = budget * (2 * table[3 * p + 2] + 1) / (dsum > 0 ? dsum : 1);
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
  CUEQ_REQUIRE(dtype == CUEQ_BF16 || dtype == CUEQ_F16 || dtype == CUEQ_F32, CUEQ_ERR_UNSUPPORTED, "linear_dw_mul_ir: bfloat16, half or float32");
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
#define DW(TI_, DM_)                                                                                                                          \
  do {                                                                                                                                        \
    auto kfn = linear_dw_mul_ir_kernel<TI_, DM_>;                                                                                                  \
    CUEQ_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kfn), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds))); \
    hipLaunchKernelGGL(kfn, dim3(static_cast<unsigned>(items)), dim3(256), lds, stream, static_cast<const TI_*>(A), lda, static_cast<const TI_*>(G), \
                       ldg, parts, nparts, partials, static_cast<int>(K), static_cast<int>(N), rows, static_cast<float>(alpha));              \
  } while (0)
#define DW_D(TI_)                                                                         \
  switch (dmax) { case 1: DW(TI_, 1); break; case 3: DW(TI_, 3); break; case 5: DW(TI_, 5); break; default: DW(TI_, 7); break; }
  if (dtype == CUEQ_F32) { DW_D(float) } else if (dtype == CUEQ_F16) { DW_D(f16bits) } else { DW_D(uint16_t) }
#undef DW_D
#undef DW
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}
