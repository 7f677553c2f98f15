// Row-streaming product for Linear-like operations on rows that keep the irrep component contiguous (`mul_ir`:
// element (channel u, component i) of a block at u * D + i), bfloat16 or float32 elements, float32 accumulation:
//   C[z, c_p + v * D + i] = alpha * sum_u A[z, a_p + u * D + i] * W_s(p)[u, v]     for every part p, all rows z, i < D.
// The reference transposes such rows to channel-contiguous ones in front of its dense kernels and back behind them
// (cuequivariance_torch/primitives/transpose.py:83-183, used by operations/linear.py:30-191); here the rows are read
// and written as they lie.
//
// Same shape of launch as linear_rows.hip (weight blocks resident in LDS, one persistent block per compute unit, every
// wavefront on its own after the weights are in place), with these differences:
//  * a unit is 16 rows of one part; it is worked on in slices of 128 * D bytes per row (64 channels of a 2-byte type, 32 of
//    float: whole 128-byte lines) which are requested ahead, pass through the wavefront's staging tile and come back as one
//    contiguous run of 32 * D bytes per lane: 16 (8) channels with all their components;
//  * the order of the contraction index inside a product is free as long as both operands agree, so the run is used as it
//    is: for float every register is one (u, i) element, for the 2-byte types the eight values of one component are picked
//    out of the run with one byte permute per register (no 2-byte LDS traffic);
//  * the products are 16 x 16 (weight columns x rows), so that the accumulators of all D components of a unit stay in
//    registers: 4 * D * N / 16 per lane - a lane ends up with 4 channels x D components of its row, which are 4 * D
//    contiguous elements of the result row and leave through the staging tile as whole lines.
// The parts of one launch may have different numbers of components D (1, 3, 5 or 7 - the irreps of one Linear).  The blocks of
// the launch are dealt out to the values of D in proportion to the bytes their parts move, and every block walks all rows for
// the parts of its D: the groups advance through the rows at the same pace, so what the chip reads and writes at one time are
// whole rows.  That matters to the memory system: launches that touch only a column range of every row measured 5.0 TB/s where
// whole rows reach 5.7.

#include "common.h"
#include "cw_common.h"
#include "u1d_spec.h"
#include "linear_rows_common.h"

namespace cueq {

namespace {

typedef float mi_floatx4 __attribute__((ext_vector_type(4)));

// WAVES: wavefronts per block, the same for all blocks of a launch (8 while the accumulators of its largest D leave room for
// two wavefronts per SIMD, else 4).
template <int DMAX, int NT16>
struct MiLaunch { static constexpr int WAVES = 4 * DMAX * NT16 <= 96 ? 8 : 4; };

template <typename TI, int D, int NT16, int WAVES_>
struct MiShape {
  static constexpr int ES = sizeof(TI);
  static constexpr int US = 128 / ES;        // channels per slice
  static constexpr int NV = 2 * D;           // 16-byte vectors per lane and slice
  static constexpr int RS = 128 * D + 16;    // bytes between the rows of the staging tile
  static constexpr int STAGE = 16 * RS;      // per wavefront
  static constexpr int ACC = 4 * D * NT16;   // accumulator registers per lane
  static constexpr int WAVES = WAVES_;
  static constexpr int TPP = 8 / ES;         // 16-column tiles of the result per pass through the staging tile
  // slices requested ahead (register sets of 8 D registers): two where the registers are tight, more for the small D of a launch
  // whose blocks run four wavefronts - about the same number of bytes in flight per wavefront either way
  static constexpr int PF = WAVES == 8 ? (D == 1 ? 4 : 2) : (D == 1 ? 8 : D == 3 ? 3 : D == 5 ? 2 : 1);
};

// one dword made of two 2-byte halves: the low half from half `lh` of `lo`, the high half from half `hh` of `hi`
template <int LH, int HH>
__device__ __forceinline__ uint32_t mi_pick(uint32_t lo, uint32_t hi) {
  constexpr uint32_t sel = (LH ? 0x0302u : 0x0100u) | ((HH ? 0x0706u : 0x0504u) << 16);
  return __builtin_amdgcn_perm(hi, lo, sel);
}

// Requests of one slice: 16 rows x 8 D vectors.  Vector v of a lane is vector 8 (v % D) + lane % 8 of row
// 8 (v / D) + lane / 8: every instruction covers one whole 128-byte line of eight rows, and the address is a part that
// depends on the lane plus a part that depends on v (kept in scalar registers / immediate offsets).  Rows past
// `last_row` repeat it.
template <int D, bool FULL>
__device__ __forceinline__ void mi_request(uint4 (&xs)[2 * D], const char* base, int row_bytes, int last_row, int lane) {
  if constexpr (FULL) {
    const char* p0 = base + (lane >> 3) * row_bytes + 16 * (lane & 7);
    const char* p1 = p0 + 8 * row_bytes;
#pragma unroll
    for (int v = 0; v < 2 * D; ++v) xs[v] = lr_stream_load((v < D ? p0 : p1) + 128 * (v % D));
  } else {
#pragma unroll
    for (int v = 0; v < 2 * D; ++v) {
      int r = 8 * (v / D) + (lane >> 3);
      r = r < last_row ? r : last_row;
      xs[v] = lr_stream_load(base + r * row_bytes + 128 * (v % D) + 16 * (lane & 7));
    }
  }
}

// The state a wavefront keeps while it walks its units.
template <typename TI, int D, int NT16>
struct MiWork {
  using S = MiShape<TI, D, NT16, 8>;  // (what it reads does not depend on the number of wavefronts)
  mi_floatx4 acc[D][NT16];

  __device__ __forceinline__ void clear() {
#pragma unroll
    for (int i = 0; i < D; ++i)
#pragma unroll
      for (int t = 0; t < NT16; ++t) acc[i][t] = mi_floatx4{0.f, 0.f, 0.f, 0.f};
  }

  // One slice: xs (as requested) -> staging tile -> the lane's run -> products with the weight rows at `wl` (the lane's
  // row c of tile 0, offset to its channels of this slice).  `refill()` may load xs again once the tile holds the slice.
  template <typename Refill>
  __device__ __forceinline__ void slice(uint4 (&xs)[2 * D], const char* wl, int WRS, char* stage, int lane, Refill&& refill) {
    constexpr int NV = S::NV, RS = S::RS, ES = S::ES;
    const int c = lane & 15, h = lane >> 4;
    {
      char* w0 = stage + (lane >> 3) * RS + 16 * (lane & 7);
#pragma unroll
      for (int v = 0; v < NV; ++v) *reinterpret_cast<uint4*>(w0 + (v / D) * (8 * RS) + 128 * (v % D)) = xs[v];
    }
    __builtin_amdgcn_wave_barrier();
    // the lane's run: 32 D bytes of row c - channels 16 h .. 16 h + 15 (2-byte type) or 8 h .. 8 h + 7 (float), D components each
    const char* rp = stage + c * RS + h * (32 * D);
    if constexpr (ES == 2) {
      uint32_t run[2][2 * NV];  // per product step: 8 channels x D components
      auto read_run = [&](int ks) {
#pragma unroll
        for (int v = 0; v < D; ++v) {
          const uint4 q = *reinterpret_cast<const uint4*>(rp + 16 * (D * ks + v));
          run[ks][4 * v] = q.x; run[ks][4 * v + 1] = q.y; run[ks][4 * v + 2] = q.z; run[ks][4 * v + 3] = q.w;
        }
      };
      read_run(0);
      __builtin_amdgcn_wave_barrier();
      refill();
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {  // elements j * D + i of the step's run: channel j (< 8), component i
        uint4 xop[D];
#pragma unroll
        for (int i = 0; i < D; ++i) {
          uint32_t w[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int e0 = 2 * j * D + i, e1 = e0 + D;  // (halves chosen at compile time: the loops are unrolled)
            const uint32_t lo = run[ks][e0 >> 1], hi = run[ks][e1 >> 1];
            w[j] = (e0 & 1) ? ((e1 & 1) ? mi_pick<1, 1>(lo, hi) : mi_pick<1, 0>(lo, hi)) : ((e1 & 1) ? mi_pick<0, 1>(lo, hi) : mi_pick<0, 0>(lo, hi));
          }
          xop[i] = make_uint4(w[0], w[1], w[2], w[3]);
        }
        if (ks == 0) read_run(1);  // (arrives while the first step multiplies)
        __builtin_amdgcn_sched_barrier(0);
        const char* wk = wl + 16 * ks;
#pragma unroll
        for (int t = 0; t < NT16; ++t) {
          const uint4 wf = *reinterpret_cast<const uint4*>(wk);
          wk += 16 * WRS;
#pragma unroll
          for (int i = 0; i < D; ++i)
            acc[i][t] = mm_16x16x32<TI>(wf, xop[i], acc[i][t]);
          if (t % 2 == 1) __builtin_amdgcn_sched_barrier(0);
        }
      }
    } else {
      uint32_t run[4 * NV];
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        const uint4 q = *reinterpret_cast<const uint4*>(rp + 16 * v);
        run[4 * v] = q.x; run[4 * v + 1] = q.y; run[4 * v + 2] = q.z; run[4 * v + 3] = q.w;
      }
      __builtin_amdgcn_wave_barrier();
      refill();
      const char* wk = wl;
#pragma unroll
      for (int t = 0; t < NT16; ++t) {
        const uint4 w0 = *reinterpret_cast<const uint4*>(wk), w1 = *reinterpret_cast<const uint4*>(wk + 16);
        wk += 16 * WRS;
        const uint32_t wv[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
          for (int i = 0; i < D; ++i)
            acc[i][t] = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(wv[j]), __uint_as_float(run[j * D + i]), acc[i][t], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  // The unit's result: lane (c, h) holds, for row c and tile t, the channels 16 t + 4 h + r (r < 4) with their D components:
  // 4 D contiguous elements of the result row.  TPP tiles at a time go through the staging tile and leave as whole lines.
  template <bool FULL>
  __device__ __forceinline__ void store(char* stage, TI* crow, int64_t ldc, int rows, float alpha, int lane) {
    constexpr int RS = S::RS, ES = S::ES, TPP = S::TPP;
    const int c = lane & 15, h = lane >> 4;
#pragma unroll
    for (int t0 = 0; t0 < NT16; t0 += TPP) {
      const int nt = NT16 - t0 < TPP ? NT16 - t0 : TPP;  // tiles of this pass
#pragma unroll
      for (int tt = 0; tt < TPP; ++tt) {
        if (tt >= nt) continue;
        char* dst = stage + c * RS + ((16 * tt + 4 * h) * D) * ES;
        float val[4 * D];
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
          for (int i = 0; i < D; ++i) val[r * D + i] = alpha * acc[i][t0 + tt][r];
        if constexpr (ES == 2) {
#pragma unroll
          for (int w = 0; w < D; ++w)
            *reinterpret_cast<uint2*>(dst + 8 * w) = make_uint2(mm_pack<TI>(val[4 * w], val[4 * w + 1]), mm_pack<TI>(val[4 * w + 2], val[4 * w + 3]));
        } else {
#pragma unroll
          for (int w = 0; w < D; ++w)
            *reinterpret_cast<float4*>(dst + 16 * w) = make_float4(val[4 * w], val[4 * w + 1], val[4 * w + 2], val[4 * w + 3]);
        }
      }
      __builtin_amdgcn_wave_barrier();
      // a pass holds nt * 16 * D * ES bytes per row = nt * D * ES / 8 lines; instruction v moves line v % lines of the rows
      // 8 (v / lines) + lane / 8 (the last line of a pass of one 2-byte tile is half a line)
      const int row_bytes_pass = nt * 16 * D * ES;
      const int lines = (row_bytes_pass + 127) / 128;
      TI* cpass = crow + t0 * 16 * D;
      const int lr = lane >> 3, lq = 16 * (lane & 7);
#pragma unroll
      for (int v = 0; v < 2 * ((16 * TPP * D * ES + 127) / 128); ++v) {
        if (v >= 2 * lines) continue;
        const int r = 8 * (v / lines) + lr, q = 128 * (v % lines) + lq;
        if (q < row_bytes_pass && (FULL || r < rows)) {
          const uint4 x = *reinterpret_cast<const uint4*>(stage + r * RS + q);
          lr_stream_store(x, reinterpret_cast<char*>(cpass + static_cast<int64_t>(r) * ldc) + q);
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
};

struct MiParts {
  int32_t a_off[kLrMaxParts], c_off[kLrMaxParts];
  int8_t slot[kLrMaxParts];  // the part's weight block, counted within its group
  int64_t w_off[kLrMaxSlots];
  // group g holds the parts of D = 2 g + 1: parts [part_first[g], part_first[g + 1]), weight blocks [slot_first[g], ...),
  // blocks of the launch [block_first[g], ...)
  int16_t part_first[5], slot_first[5], block_first[5];
};

// The work of one block for the parts of one D: block `bid` of `nblocks`, parts `first_part ...` (nparts of them), weight
// blocks `first_slot ...` (nslots of them).
template <typename TI, int D, int NT16, int WAVES_>
__device__ __forceinline__ void mi_run(const TI* __restrict__ A, int64_t lda, const TI* __restrict__ W, const MiParts& parts, int first_part,
                                       int nparts, int first_slot, int nslots, int bid, int nblocks, int w_contraction_major,
                                       TI* __restrict__ C, int64_t ldc, int M, int K, float alpha, char* smem) {
  using S = MiShape<TI, D, NT16, WAVES_>;
  constexpr int ES = S::ES, US = S::US, NV = S::NV, WAVES = S::WAVES, N = 16 * NT16, PF = S::PF;
  const int tid = threadIdx.x, lane = tid & 63, c = lane & 15, h = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int WRS = K * ES + 16;  // bytes between weight rows (one row per result column) in LDS
  const int NS = K / US;        // slices per unit

  {
    LrParts wparts;  // (the weight staging reads the block offsets only)
    for (int s = 0; s < nslots; ++s) wparts.w_off[s] = parts.w_off[first_slot + s];
    lr_stage_weights<TI, 64 * WAVES>(W, wparts, nslots, K, N, WRS, w_contraction_major, smem, tid);
  }
  __syncthreads();

  char* stage = smem + nslots * (N * WRS) + wave * S::STAGE;
  const char* wlane = smem + c * WRS + h * 32;  // the lane's channels of a slice start 32 h bytes into it (16 h or 8 h elements)
  const int nfull = M / 16;
  const int wslot = wave * nblocks + bid, nw = nblocks * WAVES;  // wavefront-major, as in linear_rows.hip
  const int step_t = nw / nparts, step_p = nw % nparts;
  const int row_bytes = static_cast<int>(lda * ES);
  const int64_t total_full = static_cast<int64_t>(nfull) * nparts;
  MiWork<TI, D, NT16> work;
  work.clear();

  if (wslot < total_full) {
    const int mine = static_cast<int>((total_full - wslot + nw - 1) / nw);  // units of this wavefront
    const int nsteps = mine * NS;                                            // slices of this wavefront
    // the slice worked on and the slice requested, each as (tile, part, slice)
    int t = wslot / nparts, p = wslot % nparts, s = 0;
    int rt = t, rp = p, rs = 0;
    auto advance = [&](int& tt, int& pp, int& ss) {
      if (++ss == NS) {
        ss = 0;
        tt += step_t;
        pp += step_p;
        if (pp >= nparts) { pp -= nparts; ++tt; }
      }
    };
    auto source = [&]() {
      const int tt = rt < nfull ? rt : nfull - 1;  // past the end: a tile that exists (the values are not used)
      return reinterpret_cast<const char*>(A + static_cast<int64_t>(tt) * 16 * lda + parts.a_off[first_part + rp]) + rs * (128 * D);
    };
    // PF register sets in rotation: the slice PF steps ahead is requested as soon as the current one sits in the staging
    // tile.  The loop body is PF steps without a branch around them; the steps left over follow it.
    uint4 xs[PF][NV];
#pragma unroll
    for (int k = 0; k < PF; ++k) {
      mi_request<D, true>(xs[k], source(), row_bytes, 15, lane);
      advance(rt, rp, rs);
    }
#define MI_STEP(XS)                                                                                                                     \
    {                                                                                                                                    \
      const char* src = source();                                                                                                        \
      work.slice(XS, wlane + parts.slot[first_part + p] * (N * WRS) + s * 128, WRS, stage, lane,                                                 \
                 [&]() { mi_request<D, true>(XS, src, row_bytes, 15, lane); __builtin_amdgcn_sched_barrier(0); });                       \
      advance(rt, rp, rs);                                                                                                               \
      if (s == NS - 1) {                                                                                                                 \
        work.template store<true>(stage, C + static_cast<int64_t>(t) * 16 * ldc + parts.c_off[first_part + p], ldc, 16, alpha, lane);            \
        work.clear();                                                                                                                    \
      }                                                                                                                                  \
      advance(t, p, s);                                                                                                                  \
    }
    for (int it = 0; it < nsteps / PF; ++it) {
#pragma unroll
      for (int k = 0; k < PF; ++k) MI_STEP(xs[k])
    }
#pragma unroll
    for (int k = 0; k < PF - 1; ++k)
      if (k < nsteps % PF) MI_STEP(xs[k])
#undef MI_STEP
  }
  if (M % 16 != 0) {  // the units of the last, partial tile
    const int rows = M - nfull * 16;
    for (int p = wslot; p < nparts; p += nw) {
      work.clear();
      for (int s = 0; s < NS; ++s) {
        uint4 xs[NV];
        mi_request<D, false>(xs, reinterpret_cast<const char*>(A + static_cast<int64_t>(nfull) * 16 * lda + parts.a_off[first_part + p]) + s * (128 * D), row_bytes,
                      rows - 1, lane);
        work.slice(xs, wlane + parts.slot[first_part + p] * (N * WRS) + s * 128, WRS, stage, lane, []() {});
      }
      work.template store<false>(stage, C + static_cast<int64_t>(nfull) * 16 * ldc + parts.c_off[first_part + p], ldc, rows, alpha, lane);
    }
  }
}


// DMAX: the largest D of the launch (it sets the wavefronts per block and the registers of the kernel).
template <typename TI, int DMAX, int NT16>
__global__ void __launch_bounds__((64 * MiLaunch<DMAX, NT16>::WAVES), 1)
    linear_rows_mul_ir_kernel(const TI* __restrict__ A, int64_t lda, const TI* __restrict__ W, MiParts parts, int w_contraction_major,
                              TI* __restrict__ C, int64_t ldc, int M, int K, float alpha) {
  constexpr int WAVES = MiLaunch<DMAX, NT16>::WAVES;
  extern __shared__ __align__(16) char smem[];
  const int b = blockIdx.x;
  int g = 0;
  while (g < 3 && b >= parts.block_first[g + 1]) ++g;
  const int bid = b - parts.block_first[g], nblocks = parts.block_first[g + 1] - parts.block_first[g];
  const int fp = parts.part_first[g], np = parts.part_first[g + 1] - fp, fs = parts.slot_first[g], ns = parts.slot_first[g + 1] - fs;
  if (g == 0) mi_run<TI, 1, NT16, WAVES>(A, lda, W, parts, fp, np, fs, ns, bid, nblocks, w_contraction_major, C, ldc, M, K, alpha, smem);
  if constexpr (DMAX >= 3) { if (g == 1) mi_run<TI, 3, NT16, WAVES>(A, lda, W, parts, fp, np, fs, ns, bid, nblocks, w_contraction_major, C, ldc, M, K, alpha, smem); }
  if constexpr (DMAX >= 5) { if (g == 2) mi_run<TI, 5, NT16, WAVES>(A, lda, W, parts, fp, np, fs, ns, bid, nblocks, w_contraction_major, C, ldc, M, K, alpha, smem); }
  if constexpr (DMAX >= 7) { if (g == 3) mi_run<TI, 7, NT16, WAVES>(A, lda, W, parts, fp, np, fs, ns, bid, nblocks, w_contraction_major, C, ldc, M, K, alpha, smem); }
}

}  // namespace

}  // namespace cueq

// table: host memory, nparts rows of (a_off, w_off, c_off, D) in elements; a part reads K * D and writes N * D elements per row
extern "C" int cueq_linear_rows_mul_ir(int32_t dtype, int32_t w_contraction_major, int64_t M, int64_t N, int64_t K, const void* A, int64_t lda,
                                       const void* W, int64_t w_numel, void* C, int64_t ldc, const int64_t* table, int64_t nparts, double alpha,
                                       void* stream_) {
  using namespace cueq;
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  CUEQ_REQUIRE(dtype == CUEQ_BF16 || dtype == CUEQ_F16 || dtype == CUEQ_F32, CUEQ_ERR_UNSUPPORTED, "linear_rows_mul_ir: bfloat16, half or float32");
  CUEQ_REQUIRE(M >= 0 && N > 0 && K > 0 && nparts >= 0, CUEQ_ERR_INVALID, "linear_rows_mul_ir: bad extents");
  const int es = dtype == CUEQ_F32 ? 4 : 2, epv = 16 / es, us = 128 / es;
  CUEQ_REQUIRE(N % 32 == 0 && N <= 128 && K % us == 0 && K <= 128, CUEQ_ERR_UNSUPPORTED,
               "linear_rows_mul_ir: N must be 32, 64, 96 or 128 and K a multiple of %d up to 128", us);
  CUEQ_REQUIRE(nparts <= kLrMaxParts, CUEQ_ERR_TOO_LARGE, "linear_rows_mul_ir: at most %d parts per launch", kLrMaxParts);
  if (M == 0 || nparts == 0) return CUEQ_OK;
  CUEQ_REQUIRE(A && W && C && table, CUEQ_ERR_INVALID, "linear_rows_mul_ir: null operand");
  CUEQ_REQUIRE(M <= (1ll << 31) - 64, CUEQ_ERR_TOO_LARGE, "linear_rows_mul_ir: too many rows");
  CUEQ_REQUIRE(lda * es < (1ll << 27) && ldc * es < (1ll << 27), CUEQ_ERR_TOO_LARGE, "linear_rows_mul_ir: rows too long");
  CUEQ_REQUIRE(lda % epv == 0 && ldc % epv == 0 && reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(C) % 16 == 0,
               CUEQ_ERR_UNSUPPORTED, "linear_rows_mul_ir: row strides and pointers must be multiples of 16 bytes");
  for (int64_t p = 0; p < nparts; ++p) {
    const int64_t a_off = table[4 * p], w_off = table[4 * p + 1], c_off = table[4 * p + 2], d = table[4 * p + 3];
    CUEQ_REQUIRE(d == 1 || d == 3 || d == 5 || d == 7, CUEQ_ERR_UNSUPPORTED, "linear_rows_mul_ir: blocks of 1, 3, 5 or 7 components");
    CUEQ_REQUIRE(a_off >= 0 && a_off + K * d <= lda && c_off >= 0 && c_off + N * d <= ldc && w_off >= 0 && w_off + K * N <= w_numel &&
                     a_off % epv == 0 && c_off % epv == 0 && w_off % epv == 0,
                 CUEQ_ERR_INVALID, "linear_rows_mul_ir: part %lld: offsets must lie inside a row / the weights and be multiples of 16 bytes",
                 static_cast<long long>(p));
  }
  // the parts grouped by D (group g: D = 2 g + 1), each group with its own list of weight blocks
  MiParts parts;
  int np = 0, nslots = 0, dmax = 1, max_slots = 0;
  int64_t weight[4] = {0, 0, 0, 0};
  for (int g = 0; g < 4; ++g) {
    parts.part_first[g] = static_cast<int16_t>(np);
    parts.slot_first[g] = static_cast<int16_t>(nslots);
    for (int64_t p = 0; p < nparts; ++p) {
      if (table[4 * p + 3] != 2 * g + 1) continue;
      const int64_t w_off = table[4 * p + 1];
      int s = parts.slot_first[g];
      while (s < nslots && parts.w_off[s] != w_off) ++s;
      if (s == nslots) {
        CUEQ_REQUIRE(nslots < kLrMaxSlots, CUEQ_ERR_TOO_LARGE, "linear_rows_mul_ir: at most %d distinct weight blocks per launch", kLrMaxSlots);
        parts.w_off[nslots++] = w_off;
      }
      parts.a_off[np] = static_cast<int32_t>(table[4 * p]);
      parts.c_off[np] = static_cast<int32_t>(table[4 * p + 2]);
      parts.slot[np] = static_cast<int8_t>(s - parts.slot_first[g]);
      ++np;
      weight[g] += 2 * g + 1;
      dmax = 2 * g + 1;
    }
    if (nslots - parts.slot_first[g] > max_slots) max_slots = nslots - parts.slot_first[g];
  }
  parts.part_first[4] = static_cast<int16_t>(np);
  parts.slot_first[4] = static_cast<int16_t>(nslots);
  if (dmax == 1) dmax = 3;  // (parts of one component alone: cueq_linear_rows is the better launch, this one still serves them)
  const int waves = 4 * dmax * (N / 16) <= 96 ? 8 : 4;
  const size_t lds = static_cast<size_t>(max_slots) * N * (es * K + 16) + static_cast<size_t>(waves) * 16 * (128 * dmax + 16);
  CUEQ_REQUIRE(lds <= 160 * 1024, CUEQ_ERR_TOO_LARGE, "linear_rows_mul_ir: the weight blocks of one launch do not fit the local data share");
  // blocks per group in proportion to the bytes its parts move (sum of D), every group with parts at least one, none more
  // than it has units for its wavefronts
  const int64_t tiles = (M + 15) / 16;
  int64_t budget = device_cus(), wsum = weight[0] + weight[1] + weight[2] + weight[3];
  int64_t nb[4], total_blocks = 0;
  for (int g = 0; g < 4; ++g) {
    const int64_t gp = parts.part_first[g + 1] - parts.part_first[g];
    nb[g] = gp == 0 ? 0 : (budget * weight[g] + wsum / 2) / wsum;
    const int64_t most = (tiles * gp + waves - 1) / waves;
    if (gp > 0 && nb[g] < 1) nb[g] = 1;
    if (nb[g] > most) nb[g] = most;
    parts.block_first[g] = static_cast<int16_t>(total_blocks);
    total_blocks += nb[g];
  }
  parts.block_first[4] = static_cast<int16_t>(total_blocks);
  KernelTimer timer("linear_rows_mul_ir", stream);
#define MI(TI_, D_, NT_)                                                                                                                      \
  do {                                                                                                                                        \
    auto kfn = linear_rows_mul_ir_kernel<TI_, D_, NT_>;                                                                                       \
    CUEQ_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kfn), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds))); \
    hipLaunchKernelGGL(kfn, dim3(static_cast<unsigned>(total_blocks)), dim3(64 * MiLaunch<D_, NT_>::WAVES), lds, stream, static_cast<const TI_*>(A), \
                       lda, static_cast<const TI_*>(W), parts, w_contraction_major, static_cast<TI_*>(C), ldc, static_cast<int>(M),           \
                       static_cast<int>(K), static_cast<float>(alpha));                                                                       \
  } while (0)
#define MI_N(TI_, D_)                                                                                                                          \
  switch (N / 32) { case 1: MI(TI_, D_, 2); break; case 2: MI(TI_, D_, 4); break; case 3: MI(TI_, D_, 6); break; default: MI(TI_, D_, 8); break; }
#define MI_D(TI_)                 \
  switch (dmax) {                 \
    case 3: MI_N(TI_, 3); break;  \
    case 5: MI_N(TI_, 5); break;  \
    default: MI_N(TI_, 7); break; \
  }
  if (dtype == CUEQ_F32) { MI_D(float) } else if (dtype == CUEQ_F16) { MI_D(f16bits) } else { MI_D(uint16_t) }
#undef MI_D
#undef MI_N
#undef MI
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}
