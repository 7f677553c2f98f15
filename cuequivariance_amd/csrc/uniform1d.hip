// uniform-1d executor: plan creation and the table-driven kernels.
//
// A plan regroups the descriptor's paths by (output buffer, output segment) and uploads
// them once.  In the table-driven kernels of this file every output element is owned by one
// thread - a lane of a wavefront that works on 64 channels of one output segment, where the output
// carries at least 32 channels - or by one wavefront when a scalar output contracts the channel
// mode; the owner walks the batch rows that contribute to it and the paths of its segment in a
// fixed order (very long rows of an indexed output in pieces that are added in order): no atomics,
// results are bit-reproducible from run to run.  (The generated channel-wise backward scatters
// the gradient of a gathered operand with floating-point atomics unless the "deterministic"
// option is set; everything else there is bit-reproducible too.)
//
// Semantics follow the reference's PyTorch executor,
// cuequivariance_torch/cuequivariance_torch/primitives/segmented_polynomial_naive.py:61-160
// (per path: coefficient * product of the operand segments, summed per output segment) and
// :376-433 (gather of indexed inputs, scatter-add of indexed outputs, sum over the batch
// for a one-row output).

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "common.h"
#include "u1d_spec.h"

namespace cueq {

static thread_local std::string g_error;

// ---- registry of specialised kernels (filled by static initialisers of generated files) ----
// (entries also arrive while the program runs: translation units compiled for a descriptor at first use register
// themselves when their shared object is loaded, possibly while another thread creates a plan)
static std::vector<const U1dSpec*>& spec_list() {
  static std::vector<const U1dSpec*> v;
  return v;
}
static std::mutex& spec_mutex() {
  static std::mutex m;
  return m;
}
static std::atomic<uint64_t> g_spec_version{1};  // bumped by every registration: plans look their entries up again
void register_u1d_spec(const U1dSpec* spec) {
  std::lock_guard<std::mutex> lock(spec_mutex());
  spec_list().push_back(spec);
  g_spec_version.fetch_add(1, std::memory_order_release);
}
static bool spec_takes(const U1dSpec* s, int io_dtype) {
  return io_dtype < 0 ? (s->io_dtype == CUEQ_F32 || s->io_dtype == CUEQ_F64) : s->io_dtype == io_dtype;
}
const U1dSpec* find_u1d_spec(uint64_t hash, int io_dtype) {
  std::lock_guard<std::mutex> lock(spec_mutex());
  for (const U1dSpec* s : spec_list())
    if (s->hash == hash && spec_takes(s, io_dtype)) return s;
  return nullptr;
}

// ---- process-wide options: the environment is read once, cueq_set_option changes them afterwards ----
static int env_flag(const char* name) {
  const char* e = getenv(name);
  return (e && e[0] == '1') ? 1 : 0;
}
static std::atomic<int>& opt_deterministic() {
  static std::atomic<int> v{env_flag("CUEQ_DETERMINISTIC")};
  return v;
}
static std::atomic<int>& opt_force_generic() {
  static std::atomic<int> v{env_flag("CUEQ_FORCE_GENERIC")};
  return v;
}
bool deterministic_scatter() { return opt_deterministic().load(std::memory_order_relaxed) != 0; }

// Groups of one segment each are the default row layout: such a buffer counts as having none (the Python table builder
// drops them the same way), so that both spellings of the same rows find the same generated kernels.
static bool has_row_layout(const cueq_u1d_desc* d, int b, int64_t first_group) {
  if (!d->layout_num_groups || d->layout_num_groups[b] <= 0) return false;
  if (!d->layout_group_dims) return true;  // (refused by cueq_u1d_plan_create)
  for (int g = 0; g < d->layout_num_groups[b]; ++g)
    if (d->layout_group_dims[first_group + g] != 1) return true;
  return false;
}

uint64_t hash_u1d_desc(const cueq_u1d_desc* d) {
  Fnv64 f;
  const int nbuf = d->num_inputs + d->num_outputs;
  f.word(static_cast<uint64_t>(d->math_dtype));
  f.word(static_cast<uint64_t>(d->operand_extent));
  f.word(static_cast<uint64_t>(d->num_inputs));
  f.word(static_cast<uint64_t>(d->num_outputs));
  for (int b = 0; b < nbuf; ++b) f.word(static_cast<uint64_t>(d->buffer_dim[b]));
  for (int b = 0; b < nbuf; ++b) f.word(static_cast<uint64_t>(d->buffer_num_segments[b]));
  f.word(static_cast<uint64_t>(d->num_operations));
  int64_t off = 0;
  for (int o = 0; o < d->num_operations; ++o) {
    const int nop = d->num_operands[o];
    f.word(static_cast<uint64_t>(nop));
    for (int k = 0; k < nop; ++k) f.word(static_cast<uint64_t>(d->operations[off + k]));
    off += nop;
    f.word(static_cast<uint64_t>(d->num_paths[o]));
    const int64_t pi0 = d->path_indices_start[o], pc0 = d->path_coefficients_start[o];
    for (int64_t i = 0; i < static_cast<int64_t>(d->num_paths[o]) * nop; ++i)
      f.word(static_cast<uint64_t>(d->path_indices[pi0 + i]));
    for (int p = 0; p < d->num_paths[o]; ++p) {
      uint64_t bits;
      std::memcpy(&bits, &d->path_coefficients[pc0 + p], 8);
      f.word(bits);
    }
  }
  // row layouts (descriptors without any hash as they always did)
  bool any_layout = false;
  if (d->layout_num_groups) {
    int64_t g0 = 0;
    for (int b = 0; b < nbuf; ++b) {
      any_layout |= has_row_layout(d, b, g0);
      g0 += d->layout_num_groups[b] > 0 ? d->layout_num_groups[b] : 0;
    }
  }
  if (any_layout) {
    f.word(0x6C61796F757473ull);
    int64_t g0 = 0;
    for (int b = 0; b < nbuf; ++b) {
      const int ng = d->layout_num_groups[b] > 0 ? d->layout_num_groups[b] : 0;
      const bool lay = has_row_layout(d, b, g0);
      f.word(static_cast<uint64_t>(lay ? ng : 0));
      for (int g = 0; lay && g < ng; ++g) f.word(static_cast<uint64_t>(d->layout_group_dims[g0 + g]));
      g0 += ng;
    }
  }
  return f.h;
}

// ---- event timing -----------------------------------------------------------------------
struct TimingRecord { const char* name; hipEvent_t start, stop; };
static std::mutex g_timing_mutex;
static bool g_timing_on = false;
static std::vector<TimingRecord> g_timing;
static thread_local hipEvent_t g_pending_start = nullptr;

bool timing_enabled() { return g_timing_on; }

void timing_mark(const char* name, hipStream_t stream, bool begin) {
  if (begin) {
    hipEvent_t e;
    if (hipEventCreate(&e) != hipSuccess) return;
    (void)hipEventRecord(e, stream);
    g_pending_start = e;
  } else if (g_pending_start) {
    hipEvent_t e;
    if (hipEventCreate(&e) != hipSuccess) return;
    (void)hipEventRecord(e, stream);
    std::lock_guard<std::mutex> lock(g_timing_mutex);
    g_timing.push_back({name, g_pending_start, e});
    g_pending_start = nullptr;
  }
}

void set_error(const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_error = buf;
}

constexpr int kMaxBuffers = 16;   // inputs + outputs of one polynomial
constexpr int kMaxInOperands = 7; // input operands of one path
constexpr int kShareChunk = 128;  // batch rows folded by one thread when an output is shared

struct DevBuffer {
  const void* data;
  const void* index;
  int64_t rows;
  int32_t dtype;
  int32_t mode;
  int32_t index_is_64;
  int32_t dim;
  int32_t nseg;
  int32_t pad;
  // row layout other than "segment s, channel u at s * extent + u": element offset of (s, u) = seg_base[s] + u * seg_stride[s]
  const int32_t* seg_base;
  const int32_t* seg_stride;
};

// One path as the wavefront-uniform kernels read it - 80 bytes in one piece (the separate arrays below cost three requests
// and leave the buffer's mode, type and layout to be looked up per operand): operand k is element off[k] + u * stride[k] of
// the row of buffer buf[k] (stride 0: a scalar operand; the row layout of the buffer is worked into off and stride).
struct PathRow {
  double coeff;
  int32_t nin;
  int32_t channel;             // 1 when one of the inputs carries the channel mode
  uint8_t buf[8];
  int32_t off[kMaxInOperands];
  int32_t stride[kMaxInOperands];
};
static_assert(sizeof(PathRow) == 80, "a path row is 80 bytes");

struct KernelArgs {
  DevBuffer buf[kMaxBuffers];
  const PathRow* rows;      // the paths once more, packed
  // path tables of the output buffer being computed
  const double* coeff;
  const int32_t* nin;       // inputs of each path
  const int32_t* in;        // [npaths * kMaxInOperands] packed (buffer << 24) | segment
  const int32_t* seg_start; // [nseg_out + 1]
  void* out;                // output tensor, or the partial buffer when chunking a shared output
  const int64_t* csr_offsets;
  const int64_t* csr_perm;
  int64_t out_rows;  // rows of `out` as addressed by this launch
  int64_t batch;
  int32_t out_dtype;
  int32_t out_mode;  // CUEQ_BATCH_*; SHARED here means "row r folds batch rows [r*chunk, (r+1)*chunk)"
  int32_t out_dim;
  int32_t out_nseg;
  int32_t extent;
  int32_t chunk;
  // an indexed output whose rows collect very many batch rows: every row is worked on in `zsplit` pieces of its range
  // (launch row c * rows_real + r = piece c of output row r, written to a partial buffer and added up in order afterwards)
  int32_t zsplit;
  int64_t rows_real;
  int32_t same_type;  // every buffer holds elements of the arithmetic type: operands are loaded without a switch on the type
  const int32_t* out_seg_base;  // layout of the output rows (null: default)
  const int32_t* out_seg_stride;
};

template <typename M>
__device__ __forceinline__ M path_product(const KernelArgs& a, int p, int64_t z, int u) {
  M prod = static_cast<M>(a.coeff[p]);
  const int n = a.nin[p];
  for (int k = 0; k < n; ++k) {
    const int32_t packed = a.in[p * kMaxInOperands + k];
    const DevBuffer& b = a.buf[packed >> 24];
    const int seg = packed & 0xffffff;
    int64_t row = 0;
    if (b.mode == CUEQ_BATCH_BATCHED) row = z;
    else if (b.mode == CUEQ_BATCH_INDEXED) row = load_index(b.index, b.index_is_64, z);
    const int64_t width = b.dim ? static_cast<int64_t>(b.nseg) * a.extent : b.nseg;
    const int64_t off = row * width + (b.dim ? (b.seg_base ? static_cast<int64_t>(b.seg_base[seg]) + static_cast<int64_t>(u) * b.seg_stride[seg]
                                                              : static_cast<int64_t>(seg) * a.extent + u)
                                            : seg);
    prod *= load_as<M>(b.data, b.dtype, off);
  }
  return prod;
}

template <typename M>
__device__ __forceinline__ void z_range(const KernelArgs& a, int64_t r, int64_t& z0, int64_t& z1) {
  if (a.out_mode == CUEQ_BATCH_BATCHED) { z0 = r; z1 = r + 1; }
  else if (a.out_mode == CUEQ_BATCH_INDEXED) {
    if (a.zsplit > 1) {
      const int64_t rr = r % a.rows_real, c = r / a.rows_real;
      const int64_t lo = a.csr_offsets[rr], len = a.csr_offsets[rr + 1] - lo;
      z0 = lo + len * c / a.zsplit;
      z1 = lo + len * (c + 1) / a.zsplit;
    } else {
      z0 = a.csr_offsets[r];
      z1 = a.csr_offsets[r + 1];
    }
  }
  else { z0 = r * a.chunk; z1 = min(z0 + a.chunk, a.batch); }
}

// One thread per output element (row, segment, channel).
template <typename M>
__global__ void __launch_bounds__(256) u1d_generic_elem(KernelArgs a) {
  const int ext_out = a.out_dim ? a.extent : 1;
  const int64_t per_row = static_cast<int64_t>(a.out_nseg) * ext_out;
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tid >= a.out_rows * per_row) return;
  const int64_t r = tid / per_row;
  const int rem = static_cast<int>(tid - r * per_row);
  const int s = rem / ext_out, u = rem - s * ext_out;
  int64_t z0, z1;
  z_range<M>(a, r, z0, z1);
  const int p0 = a.seg_start[s], p1 = a.seg_start[s + 1];
  M acc = 0;
  for (int64_t zz = z0; zz < z1; ++zz) {
    const int64_t z = (a.out_mode == CUEQ_BATCH_INDEXED) ? a.csr_perm[zz] : zz;
    for (int p = p0; p < p1; ++p) acc += path_product<M>(a, p, z, u);
  }
  const int64_t where = a.out_seg_base ? r * per_row + a.out_seg_base[s] + static_cast<int64_t>(u) * a.out_seg_stride[s] : tid;
  store_as<M>(a.out, a.out_dtype, where, acc);
}

// The product of one path for the lanes of a wavefront that differ in the channel only (`u`; p, z the same for all lanes):
// tables, batch modes, indices and row addresses are then scalar work and a path costs one load per operand and lane.
template <typename M>
__device__ __forceinline__ M path_product_lanes(const KernelArgs& a, int p, int64_t z, int u) {
  M prod = static_cast<M>(a.coeff[p]);
  const int n = a.nin[p];
  for (int k = 0; k < n; ++k) {
    const int32_t packed = a.in[p * kMaxInOperands + k];
    const DevBuffer& b = a.buf[packed >> 24];
    const int seg = packed & 0xffffff;
    int64_t row = 0;
    if (b.mode == CUEQ_BATCH_BATCHED) row = z;
    else if (b.mode == CUEQ_BATCH_INDEXED) row = load_index(b.index, b.index_is_64, z);
    if (b.dim) {
      const int64_t base = row * (static_cast<int64_t>(b.nseg) * a.extent);
      const int64_t off = b.seg_base ? base + b.seg_base[seg] + static_cast<int64_t>(u) * b.seg_stride[seg] : base + static_cast<int64_t>(seg) * a.extent + u;
      prod *= load_as<M>(b.data, b.dtype, off);
    } else {
      prod *= load_as<M>(b.data, b.dtype, row * b.nseg + seg);  // (one value for the wavefront)
    }
  }
  return prod;
}

// Path row p, the same for the whole wavefront, read through the constant address space: the table is written once when the
// plan is made and never by a kernel, so the read may go through the scalar unit into scalar registers (read as ordinary global
// memory it costs every lane a vector load, and a readfirstlane per field).
__device__ __forceinline__ PathRow load_path_row(const PathRow* rows, int p) {
  typedef const __attribute__((address_space(4))) uint32_t* ConstWords;
  ConstWords q = (ConstWords)(reinterpret_cast<uintptr_t>(rows + p));
  uint32_t w[sizeof(PathRow) / 4];
#pragma unroll
  for (int k = 0; k < static_cast<int>(sizeof(PathRow) / 4); ++k) w[k] = q[k];
  PathRow r;
  __builtin_memcpy(&r, w, sizeof(PathRow));
  return r;
}

// The row of every buffer for batch row z as a pointer, one lane per buffer, into `srow` (LDS, private to the wavefront): the
// batch mode and the index of a buffer are looked at once per batch row, not once per path and operand.  Every buffer holds
// elements of type M here (KernelArgs::same_type).
// (The pointers are kept as pointers into global memory: a load through a generic pointer counts as an LDS access as well, and the
// wait for the next row pointer would then wait for the operand loads in flight.)
template <typename M>
using GlobalRow = const __attribute__((address_space(1))) M*;

template <typename M>
__device__ __forceinline__ void row_pointers(const KernelArgs& a, int64_t z, int lane, GlobalRow<M>* srow) {
  if (lane < kMaxBuffers) {
    const DevBuffer& b = a.buf[lane];
    int64_t row = 0;
    if (b.mode == CUEQ_BATCH_BATCHED) row = z;
    else if (b.mode == CUEQ_BATCH_INDEXED && b.index != nullptr) row = load_index(b.index, b.index_is_64, z);
    srow[lane] = (GlobalRow<M>)(reinterpret_cast<uintptr_t>(b.data)) + row * (b.dim ? static_cast<int64_t>(b.nseg) * a.extent : static_cast<int64_t>(b.nseg));
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // (the same wavefront reads what it wrote: LDS works in order)
  __builtin_amdgcn_wave_barrier();
}

// One wavefront per (output row, output segment, 64 channels) of an output that carries the channel mode: the lanes are
// the channels, everything else is the same for the whole wavefront (its number is read into a scalar register, so that the
// compiler keeps tables, modes and row addresses in scalar registers).
template <typename M>
__global__ void __launch_bounds__(256) u1d_generic_rowseg(KernelArgs a) {
  const int lane = threadIdx.x & 63;
  const int wv = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int64_t wid = static_cast<int64_t>(blockIdx.x) * 4 + wv;
  const int nuc = (a.extent + 63) / 64;
  if (wid >= a.out_rows * a.out_nseg * nuc) return;
  const int uc = static_cast<int>(wid % nuc);
  const int64_t rs = wid / nuc;
  const int s = static_cast<int>(rs % a.out_nseg);
  const int64_t r = rs / a.out_nseg;
  const int u = uc * 64 + lane;
  const int ul = u < a.extent ? u : a.extent - 1;  // (lanes past the extent compute the last channel again and store nothing)
  int64_t z0, z1;
  z_range<M>(a, r, z0, z1);
  const int p0 = a.seg_start[s], p1 = a.seg_start[s + 1];
  M acc = 0;
  for (int64_t zz = z0; zz < z1; ++zz) {
    const int64_t z = (a.out_mode == CUEQ_BATCH_INDEXED) ? a.csr_perm[zz] : zz;
    for (int p = p0; p < p1; ++p) acc += path_product_lanes<M>(a, p, z, ul);
  }
  if (u < a.extent) {
    const int64_t per_row = static_cast<int64_t>(a.out_nseg) * a.extent;
    const int64_t where = a.out_seg_base ? r * per_row + a.out_seg_base[s] + static_cast<int64_t>(u) * a.out_seg_stride[s]
                                         : r * per_row + static_cast<int64_t>(s) * a.extent + u;
    store_as<M>(a.out, a.out_dtype, where, acc);
  }
}

// 1 in global memory: what the operands past the last one of a path read in u1d_rowseg_paths.
__device__ const float kOneFloat = 1.0f;
__device__ const double kOneDouble = 1.0;
template <typename M>
__device__ __forceinline__ GlobalRow<M> pointer_to_one() {
  if constexpr (sizeof(M) == 8) return (GlobalRow<M>)(reinterpret_cast<uintptr_t>(&kOneDouble));
  else return (GlobalRow<M>)(reinterpret_cast<uintptr_t>(&kOneFloat));
}

template <typename M, int N>
__device__ __forceinline__ void request_operands(const PathRow& r, int u, const GlobalRow<M>* srow, M (&v)[N]) {
#pragma unroll
  for (int k = 0; k < N; ++k) v[k] = srow[r.buf[k]][r.off[k] + u * r.stride[k]];
}

template <typename M, int N>
__device__ __forceinline__ M product_of(const PathRow& r, const M (&v)[N]) {
  M prod = static_cast<M>(r.coeff);
#pragma unroll
  for (int k = 0; k < N; ++k) prod *= v[k];
  return prod;
}

// The paths p0 <= p < p1 (p0 < p1) of one batch row for the lanes of a wavefront, every path read as exactly N operands (N: the
// most operands of a path of this output; a path with fewer has the rest point at a 1 in memory - multiplying by 1 changes no
// bit).  With the count fixed there is no branch in the walk, and the operands of a path are requested while the path before it
// still waits for its own: two paths in flight per wavefront, where the memory latency of one (row pointer from LDS, then the
// operand from L2) is what a path costs.  Returns acc + the products in the order of the table.  Reduce: the lanes are summed
// afterwards, so a path adds only where it should count - in the lanes inside the extent when it carries the channel mode,
// in the first lane of the first 64 channels otherwise.
template <typename M, int N, bool Reduce>
__device__ __forceinline__ M walk_paths(const PathRow* rows, int p0, int p1, int u, bool inside, bool first, const GlobalRow<M>* srow,
                                        M acc) {
  PathRow ra = load_path_row(rows, p0);
  PathRow rb = load_path_row(rows, p0 + 1 < p1 ? p0 + 1 : p0);
  M va[N], vb[N];
  request_operands<M, N>(ra, u, srow, va);
  for (int p = p0; p < p1; p += 2) {  // ra, va: path p; rb: path p + 1 (or the last path once more, then not added)
    request_operands<M, N>(rb, u, srow, vb);
    __builtin_amdgcn_sched_barrier(0);  // (a scalar read asked for earlier would be waited for together with the LDS reads)
    const PathRow rn = load_path_row(rows, p + 2 < p1 ? p + 2 : p1 - 1);
    const M one = product_of<M, N>(ra, va);
    acc += !Reduce || (ra.channel ? inside : first) ? one : static_cast<M>(0);
    request_operands<M, N>(rn, u, srow, va);
    __builtin_amdgcn_sched_barrier(0);
    const PathRow rm = load_path_row(rows, p + 3 < p1 ? p + 3 : p1 - 1);
    const M two = product_of<M, N>(rb, vb);
    acc += p + 1 < p1 && (!Reduce || (rb.channel ? inside : first)) ? two : static_cast<M>(0);
    ra = rn;
    rb = rm;
  }
  return acc;
}

// u1d_generic_rowseg for buffers that all hold the math type (walk_paths).
template <typename M, int N>
__global__ void __launch_bounds__(256) u1d_rowseg_paths(KernelArgs a) {
  const int lane = threadIdx.x & 63;
  const int wv = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int64_t wid = static_cast<int64_t>(blockIdx.x) * 4 + wv;
  const int nuc = (a.extent + 63) / 64;
  if (wid >= a.out_rows * a.out_nseg * nuc) return;
  const int uc = static_cast<int>(wid % nuc);
  const int64_t rs = wid / nuc;
  const int s = static_cast<int>(rs % a.out_nseg);
  const int64_t r = rs / a.out_nseg;
  const int u = uc * 64 + lane;
  const int ul = u < a.extent ? u : a.extent - 1;
  int64_t z0, z1;
  z_range<M>(a, r, z0, z1);
  const int p0 = a.seg_start[s], p1 = a.seg_start[s + 1];
  __shared__ GlobalRow<M> srow_all[4][kMaxBuffers + 1];
  GlobalRow<M>* srow = srow_all[wv];
  M acc = 0;
  if (p0 < p1) {
    for (int64_t zz = z0; zz < z1; ++zz) {
      const int64_t z = (a.out_mode == CUEQ_BATCH_INDEXED) ? a.csr_perm[zz] : zz;
      if (lane == kMaxBuffers) srow[kMaxBuffers] = pointer_to_one<M>();
      row_pointers<M>(a, z, lane, srow);
      acc = walk_paths<M, N, false>(a.rows, p0, p1, ul, true, true, srow, acc);
      __builtin_amdgcn_wave_barrier();  // (the next batch row overwrites the pointers)
    }
  }
  if (u < a.extent) {
    const int64_t per_row = static_cast<int64_t>(a.out_nseg) * a.extent;
    const int64_t where = a.out_seg_base ? r * per_row + a.out_seg_base[s] + static_cast<int64_t>(u) * a.out_seg_stride[s]
                                         : r * per_row + static_cast<int64_t>(s) * a.extent + u;
    store_as<M>(a.out, a.out_dtype, where, acc);
  }
}

// u1d_generic_wave for buffers that all hold the math type: per batch row the channels 64 at a time, all paths for each
// (walk_paths), then the butterfly over the lanes.
template <typename M, int N>
__global__ void __launch_bounds__(256) u1d_reduce_paths(KernelArgs a) {
  const int lane = threadIdx.x & 63;
  const int wv = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int64_t wid = static_cast<int64_t>(blockIdx.x) * 4 + wv;
  if (wid >= a.out_rows * a.out_nseg) return;
  const int64_t r = wid / a.out_nseg;
  const int s = static_cast<int>(wid - r * a.out_nseg);
  int64_t z0, z1;
  z_range<M>(a, r, z0, z1);
  const int p0 = a.seg_start[s], p1 = a.seg_start[s + 1];
  __shared__ GlobalRow<M> srow_all[4][kMaxBuffers + 1];
  GlobalRow<M>* srow = srow_all[wv];
  M acc = 0;
  if (p0 < p1) {
    for (int64_t zz = z0; zz < z1; ++zz) {
      const int64_t z = (a.out_mode == CUEQ_BATCH_INDEXED) ? a.csr_perm[zz] : zz;
      if (lane == kMaxBuffers) srow[kMaxBuffers] = pointer_to_one<M>();
      row_pointers<M>(a, z, lane, srow);
      for (int u0 = 0; u0 < a.extent; u0 += 64) {  // (at least once: the extent is at least 1)
        const int u = u0 + lane;
        acc = walk_paths<M, N, true>(a.rows, p0, p1, u < a.extent ? u : a.extent - 1, u < a.extent, u == 0, srow, acc);
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
  for (int d = 32; d >= 1; d >>= 1) acc += __shfl_xor(acc, d, 64);
  if (lane == 0) store_as<M>(a.out, a.out_dtype, wid, acc);
}

// One wavefront per scalar output element (row, segment): lanes stride over the channel
// mode, then a fixed-shape butterfly reduction.
template <typename M>
__global__ void __launch_bounds__(256) u1d_generic_wave(KernelArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t wid = static_cast<int64_t>(blockIdx.x) * 4 + __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  if (wid >= a.out_rows * a.out_nseg) return;
  const int64_t r = wid / a.out_nseg;
  const int s = static_cast<int>(wid - r * a.out_nseg);
  int64_t z0, z1;
  z_range<M>(a, r, z0, z1);
  const int p0 = a.seg_start[s], p1 = a.seg_start[s + 1];
  M acc = 0;
  for (int64_t zz = z0; zz < z1; ++zz) {
    const int64_t z = (a.out_mode == CUEQ_BATCH_INDEXED) ? a.csr_perm[zz] : zz;
    for (int p = p0; p < p1; ++p) {
      // a path sums over the channel mode only when one of its inputs carries it; a path of scalars contributes once
      bool has_channel = false;
      for (int k = 0; k < a.nin[p]; ++k) has_channel |= a.buf[a.in[p * kMaxInOperands + k] >> 24].dim != 0;
      if (has_channel) {
        for (int u0 = 0; u0 < a.extent; u0 += 64) {  // (u0 the same for all lanes; a lane past the extent adds nothing)
          const int u = u0 + lane;
          const M v = path_product_lanes<M>(a, p, z, u < a.extent ? u : a.extent - 1);
          acc += u < a.extent ? v : static_cast<M>(0);
        }
      } else {
        const M v = path_product_lanes<M>(a, p, z, 0);
        acc += lane == 0 ? v : static_cast<M>(0);
      }
    }
  }
  for (int d = 32; d >= 1; d >>= 1) acc += __shfl_xor(acc, d, 64);
  if (lane == 0) store_as<M>(a.out, a.out_dtype, wid, acc);
}

// out[e] = sum over chunks c (ascending) of partial[c, e]
template <typename M>
__global__ void __launch_bounds__(256) u1d_fold_chunks(const M* partial, int64_t nchunks, int64_t width, void* out,
                                                       int out_dtype) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (e >= width) return;
  M acc = 0;
  for (int64_t c = 0; c < nchunks; ++c) acc += partial[c * width + e];
  store_as<M>(out, out_dtype, e, acc);
}

struct OutTables {
  int32_t npaths = 0;
  double* coeff = nullptr;
  int32_t* nin = nullptr;
  int32_t* in = nullptr;
  PathRow* rows = nullptr;
  int32_t* seg_start = nullptr;
  int max_nin = 1;                 // the most input operands of a path (at least 1)
  bool contracts_channel = false;  // scalar output fed by channel-carrying inputs
};

}  // namespace cueq

using namespace cueq;

struct cueq_u1d_plan {
  int32_t math_dtype;
  int32_t extent;
  int32_t num_inputs, num_outputs;
  std::vector<int32_t> buffer_dim, buffer_nseg;
  std::vector<OutTables> out;  // one per output buffer
  std::vector<const int32_t*> seg_base, seg_stride;  // per buffer, device pointers (null: default layout)
  // descriptor-specialised kernels registered for these tables (one entry per element type of the buffers); looked up again
  // whenever the registry has grown since, because units compiled at first use arrive while plans exist
  static constexpr int kMaxSpecs = 4;
  mutable std::atomic<const cueq::U1dSpec*> specs[kMaxSpecs] = {};
  mutable std::atomic<int> nspecs{0};
  mutable std::atomic<uint64_t> specs_version{0};
  uint64_t hash = 0;
  void* device_blob = nullptr;
  int device = 0;
};

// Number of entries of plan->specs, after looking them up again when the registry has changed since the last look.
static int plan_specs(const cueq_u1d_plan* plan) {
  const uint64_t now = g_spec_version.load(std::memory_order_acquire);
  if (plan->specs_version.load(std::memory_order_acquire) != now) {
    std::lock_guard<std::mutex> lock(spec_mutex());
    int n = 0;  // (the registry only grows and keeps its order: entries already published keep their place)
    for (const U1dSpec* sp : spec_list())
      if (sp->hash == plan->hash && n < cueq_u1d_plan::kMaxSpecs) plan->specs[n++].store(sp, std::memory_order_relaxed);
    plan->nspecs.store(n, std::memory_order_release);
    plan->specs_version.store(g_spec_version.load(std::memory_order_acquire), std::memory_order_release);
  }
  return plan->nspecs.load(std::memory_order_acquire);
}

extern "C" const char* cueq_last_error(void) { return g_error.c_str(); }

extern "C" int cueq_timing_begin(void) {
  std::lock_guard<std::mutex> lock(g_timing_mutex);
  for (auto& r : g_timing) { (void)hipEventDestroy(r.start); (void)hipEventDestroy(r.stop); }
  g_timing.clear();
  g_timing_on = true;
  return CUEQ_OK;
}

extern "C" int cueq_timing_end(cueq_timing_entry* out, int max_entries) {
  std::lock_guard<std::mutex> lock(g_timing_mutex);
  g_timing_on = false;
  int n = 0;
  for (auto& r : g_timing) {
    float ms = 0.f;
    if (hipEventSynchronize(r.stop) == hipSuccess && hipEventElapsedTime(&ms, r.start, r.stop) == hipSuccess) {
      int k = 0;
      for (; k < n; ++k) if (std::strcmp(out[k].name, r.name) == 0) break;
      if (k == n) {
        if (n >= max_entries) { k = -1; }
        else { std::snprintf(out[n].name, sizeof(out[n].name), "%s", r.name); out[n].launches = 0; out[n].total_ms = 0; ++n; }
      }
      if (k >= 0) { out[k].launches += 1; out[k].total_ms += ms; }
    }
    (void)hipEventDestroy(r.start);
    (void)hipEventDestroy(r.stop);
  }
  g_timing.clear();
  return n;
}
extern "C" const char* cueq_version(void) { return "cueq_amd 0.1 (gfx950)"; }

extern "C" int cueq_set_option(const char* name, int32_t value) {
  CUEQ_REQUIRE(name, CUEQ_ERR_INVALID, "null option name");
  if (std::strcmp(name, "deterministic") == 0) opt_deterministic().store(value ? 1 : 0);
  else if (std::strcmp(name, "force_generic") == 0) opt_force_generic().store(value ? 1 : 0);
  else CUEQ_REQUIRE(false, CUEQ_ERR_INVALID, "unknown option '%s' (deterministic, force_generic)", name);
  return CUEQ_OK;
}
extern "C" int cueq_get_option(const char* name) {
  if (name && std::strcmp(name, "deterministic") == 0) return opt_deterministic().load();
  if (name && std::strcmp(name, "force_generic") == 0) return opt_force_generic().load();
  return -1;
}

extern "C" int cueq_u1d_plan_create(const cueq_u1d_desc* d, cueq_u1d_plan** out_plan) {
  CUEQ_REQUIRE(d && out_plan, CUEQ_ERR_INVALID, "null argument");
  CUEQ_REQUIRE(d->math_dtype == CUEQ_F32 || d->math_dtype == CUEQ_F64, CUEQ_ERR_INVALID,
               "math_dtype must be f32 or f64");
  const int nbuf = d->num_inputs + d->num_outputs;
  CUEQ_REQUIRE(d->num_inputs >= 0 && d->num_outputs >= 1 && nbuf <= kMaxBuffers, CUEQ_ERR_UNSUPPORTED,
               "polynomial has %d buffers, at most %d are supported", nbuf, kMaxBuffers);
  CUEQ_REQUIRE(d->operand_extent >= 1 && d->operand_extent < (1 << 24), CUEQ_ERR_INVALID, "bad operand_extent");
  for (int b = 0; b < nbuf; ++b) {
    CUEQ_REQUIRE(d->buffer_dim[b] == 0 || d->buffer_dim[b] == 1, CUEQ_ERR_INVALID, "buffer_dim must be 0 or 1");
    CUEQ_REQUIRE(d->buffer_num_segments[b] >= 0 && d->buffer_num_segments[b] < (1 << 24), CUEQ_ERR_INVALID,
                 "bad segment count for buffer %d", b);
  }

  struct HostPath { int out_seg; double c; int nin; int32_t in[kMaxInOperands]; };
  std::vector<std::vector<HostPath>> per_out(d->num_outputs);
  std::vector<bool> contracts(d->num_outputs, false);

  int64_t op_off = 0;
  for (int o = 0; o < d->num_operations; ++o) {
    const int nop = d->num_operands[o];
    CUEQ_REQUIRE(nop >= 1 && nop <= kMaxInOperands + 1, CUEQ_ERR_UNSUPPORTED, "operation %d has %d operands", o, nop);
    const int32_t* bufs = d->operations + op_off;
    op_off += nop;
    int out_pos = -1;
    for (int k = 0; k < nop; ++k) {
      CUEQ_REQUIRE(bufs[k] >= 0 && bufs[k] < nbuf, CUEQ_ERR_INVALID, "operation %d: buffer id out of range", o);
      if (bufs[k] >= d->num_inputs) {
        CUEQ_REQUIRE(out_pos < 0, CUEQ_ERR_INVALID, "operation %d has more than one output buffer", o);
        out_pos = k;
      }
    }
    CUEQ_REQUIRE(out_pos >= 0, CUEQ_ERR_INVALID, "operation %d has no output buffer", o);
    const int ob = bufs[out_pos] - d->num_inputs;
    const int64_t pi0 = d->path_indices_start[o], pc0 = d->path_coefficients_start[o];
    CUEQ_REQUIRE(pi0 >= 0 && pi0 + static_cast<int64_t>(d->num_paths[o]) * nop <= d->path_indices_len &&
                     pc0 >= 0 && pc0 + d->num_paths[o] <= d->path_coefficients_len,
                 CUEQ_ERR_INVALID, "operation %d: path tables out of range", o);
    for (int p = 0; p < d->num_paths[o]; ++p) {
      HostPath hp{};
      hp.c = d->path_coefficients[pc0 + p];
      hp.nin = 0;
      for (int k = 0; k < nop; ++k) {
        const int seg = d->path_indices[pi0 + static_cast<int64_t>(p) * nop + k];
        CUEQ_REQUIRE(seg >= 0 && seg < d->buffer_num_segments[bufs[k]], CUEQ_ERR_INVALID,
                     "operation %d path %d: segment %d out of range for buffer %d", o, p, seg, bufs[k]);
        if (k == out_pos) hp.out_seg = seg;
        else {
          hp.in[hp.nin++] = (bufs[k] << 24) | seg;
          if (d->buffer_dim[bufs[k]] == 1 && d->buffer_dim[bufs[out_pos]] == 0 && d->operand_extent > 1)
            contracts[ob] = true;
        }
      }
      per_out[ob].push_back(hp);
    }
  }

  auto* plan = new cueq_u1d_plan();
  plan->math_dtype = d->math_dtype;
  plan->extent = static_cast<int32_t>(d->operand_extent);
  plan->num_inputs = d->num_inputs;
  plan->num_outputs = d->num_outputs;
  plan->buffer_dim.assign(d->buffer_dim, d->buffer_dim + nbuf);
  plan->buffer_nseg.assign(d->buffer_num_segments, d->buffer_num_segments + nbuf);
  plan->out.resize(d->num_outputs);
  if (hipGetDevice(&plan->device) != hipSuccess) plan->device = 0;

  // Lay all tables out in one host blob, then one upload.
  size_t total = 0;
  auto reserve = [&](size_t bytes) { size_t o = total; total += (bytes + 15) & ~size_t(15); return o; };
  struct Off { size_t coeff, nin, in, rows, seg; };
  std::vector<Off> offs(d->num_outputs);
  for (int ob = 0; ob < d->num_outputs; ++ob) {
    auto& v = per_out[ob];
    std::stable_sort(v.begin(), v.end(), [](const HostPath& x, const HostPath& y) { return x.out_seg < y.out_seg; });
    const int nseg = d->buffer_num_segments[d->num_inputs + ob];
    offs[ob].coeff = reserve(v.size() * sizeof(double));
    offs[ob].nin = reserve(v.size() * sizeof(int32_t));
    offs[ob].in = reserve(v.size() * kMaxInOperands * sizeof(int32_t));
    offs[ob].rows = reserve((v.size() + 1) * sizeof(PathRow));
    offs[ob].seg = reserve((nseg + 1) * sizeof(int32_t));
  }
  // row layouts: per buffer the base offset and channel stride of every segment
  std::vector<size_t> lay_off(nbuf, SIZE_MAX);
  std::vector<std::vector<int32_t>> lay_tab(nbuf);
  if (d->layout_num_groups) {
    int64_t g0 = 0;
    for (int b = 0; b < nbuf; ++b) {
      const int ng = d->layout_num_groups[b];
      if (ng < 0) { delete plan; CUEQ_REQUIRE(false, CUEQ_ERR_INVALID, "negative group count for buffer %d", b); }
      if (ng > 0) {
        const int nseg = d->buffer_num_segments[b];
        std::vector<int32_t>& t = lay_tab[b];
        t.assign(2 * static_cast<size_t>(nseg), 0);
        int64_t seg = 0, off = 0;
        bool ok = d->buffer_dim[b] == 1 && d->layout_group_dims != nullptr;
        for (int g = 0; ok && g < ng; ++g) {
          const int dim = d->layout_group_dims[g0 + g];
          if (dim < 1 || seg + dim > nseg) { ok = false; break; }
          for (int c = 0; c < dim; ++c) { t[seg + c] = static_cast<int32_t>(off + c); t[nseg + seg + c] = dim; }
          seg += dim;
          off += static_cast<int64_t>(dim) * d->operand_extent;
        }
        if (!ok || seg != nseg || off >= (int64_t(1) << 31)) {
          delete plan;
          CUEQ_REQUIRE(false, CUEQ_ERR_INVALID, "layout groups of buffer %d do not partition its %d channel segments", b, nseg);
        }
        if (has_row_layout(d, b, g0)) lay_off[b] = reserve(t.size() * sizeof(int32_t));  // (groups of one segment: the default rows)
      }
      g0 += ng;
    }
  }
  std::vector<char> host(total ? total : 16, 0);
  for (int b = 0; b < nbuf; ++b)
    if (lay_off[b] != SIZE_MAX) std::memcpy(host.data() + lay_off[b], lay_tab[b].data(), lay_tab[b].size() * sizeof(int32_t));
  for (int ob = 0; ob < d->num_outputs; ++ob) {
    auto& v = per_out[ob];
    const int nseg = d->buffer_num_segments[d->num_inputs + ob];
    auto* coeff = reinterpret_cast<double*>(host.data() + offs[ob].coeff);
    auto* nin = reinterpret_cast<int32_t*>(host.data() + offs[ob].nin);
    auto* in = reinterpret_cast<int32_t*>(host.data() + offs[ob].in);
    auto* seg = reinterpret_cast<int32_t*>(host.data() + offs[ob].seg);
    auto* rows = reinterpret_cast<PathRow*>(host.data() + offs[ob].rows);
    std::vector<int32_t> count(nseg + 1, 0);
    for (size_t p = 0; p < v.size(); ++p) {
      coeff[p] = v[p].c;
      nin[p] = v[p].nin;
      std::memcpy(in + p * kMaxInOperands, v[p].in, sizeof(v[p].in));
      rows[p].coeff = v[p].c;
      rows[p].nin = v[p].nin;
      rows[p].channel = 0;
      for (int k = v[p].nin; k < kMaxInOperands; ++k) rows[p].buf[k] = kMaxBuffers;  // (the slot of the 1; offset and stride 0)
      for (int k = 0; k < v[p].nin; ++k) {
        const int bi = v[p].in[k] >> 24, sg = v[p].in[k] & 0xffffff;
        rows[p].buf[k] = static_cast<uint8_t>(bi);
        if (d->buffer_dim[bi] == 0) {  // a scalar per segment
          rows[p].off[k] = sg;
          rows[p].stride[k] = 0;
        } else if (lay_off[bi] != SIZE_MAX) {  // rows in groups: base and channel stride of the segment
          rows[p].off[k] = lay_tab[bi][sg];
          rows[p].stride[k] = lay_tab[bi][d->buffer_num_segments[bi] + sg];
          rows[p].channel = 1;
        } else {
          rows[p].off[k] = sg * static_cast<int32_t>(d->operand_extent);
          rows[p].stride[k] = 1;
          rows[p].channel = 1;
        }
      }
      count[v[p].out_seg + 1]++;
    }
    seg[0] = 0;
    for (int s = 0; s < nseg; ++s) seg[s + 1] = seg[s] + count[s + 1];
  }
  hipError_t e = hipMalloc(&plan->device_blob, host.size());
  if (e == hipSuccess) e = hipMemcpy(plan->device_blob, host.data(), host.size(), hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    set_error("uploading plan tables failed: %s", hipGetErrorString(e));
    if (plan->device_blob) (void)hipFree(plan->device_blob);
    delete plan;
    return CUEQ_ERR_HIP;
  }
  char* base = static_cast<char*>(plan->device_blob);
  for (int ob = 0; ob < d->num_outputs; ++ob) {
    OutTables& t = plan->out[ob];
    t.npaths = static_cast<int32_t>(per_out[ob].size());
    t.coeff = reinterpret_cast<double*>(base + offs[ob].coeff);
    t.nin = reinterpret_cast<int32_t*>(base + offs[ob].nin);
    t.in = reinterpret_cast<int32_t*>(base + offs[ob].in);
    t.rows = reinterpret_cast<PathRow*>(base + offs[ob].rows);
    t.seg_start = reinterpret_cast<int32_t*>(base + offs[ob].seg);
    t.contracts_channel = contracts[ob];
    for (const auto& path : per_out[ob]) t.max_nin = std::max<int>(t.max_nin, path.nin);
  }
  plan->seg_base.assign(nbuf, nullptr);
  plan->seg_stride.assign(nbuf, nullptr);
  for (int b = 0; b < nbuf; ++b)
    if (lay_off[b] != SIZE_MAX) {
      plan->seg_base[b] = reinterpret_cast<const int32_t*>(base + lay_off[b]);
      plan->seg_stride[b] = plan->seg_base[b] + d->buffer_num_segments[b];
    }
  plan->hash = hash_u1d_desc(d);
  (void)plan_specs(plan);
  *out_plan = plan;
  return CUEQ_OK;
}

// 1 when kernels generated for these tables are registered for buffers of `io_dtype` (a CUEQ_* code), else 0.  Host-only.
extern "C" int cueq_u1d_desc_serves(const cueq_u1d_desc* d, int32_t io_dtype) {
  if (!d || io_dtype < 0) return 0;
  return find_u1d_spec(hash_u1d_desc(d), io_dtype) ? 1 : 0;
}

// Host-only: content hash of the descriptor tables and whether specialised kernels are linked in.
extern "C" int cueq_u1d_desc_info(const cueq_u1d_desc* d, uint64_t* hash) {
  if (!d) return 0;
  const uint64_t h = hash_u1d_desc(d);
  if (hash) *hash = h;
  return find_u1d_spec(h) ? 1 : 0;
}

// 1 when descriptor-specialised kernels exist for this plan, else 0; *hash receives the table hash.
extern "C" int cueq_u1d_plan_info(const cueq_u1d_plan* plan, uint64_t* hash) {
  if (!plan) return 0;
  if (hash) *hash = plan->hash;
  const int n = plan_specs(plan);
  for (int i = 0; i < n; ++i)
    if (spec_takes(plan->specs[i].load(std::memory_order_relaxed), -1)) return 1;
  return 0;
}

extern "C" void cueq_u1d_plan_destroy(cueq_u1d_plan* plan) {
  if (!plan) return;
  if (plan->device_blob) (void)hipFree(plan->device_blob);
  delete plan;
}

static int64_t share_chunks(int64_t batch) { return (batch + kShareChunk - 1) / kShareChunk; }

// Pieces per row of an indexed output: 1 unless its rows collect a thousand batch rows and more on average (a weight
// gradient indexed by a handful of classes: few rows, hence few wavefronts, each with a long walk), then about 64 batch rows a
// piece, at most 64 pieces.
static int64_t row_splits(int64_t batch, int64_t rows) {
  if (rows <= 0 || batch / rows < 1024) return 1;
  return std::min<int64_t>(64, (batch / rows + 63) / 64);
}

extern "C" int64_t cueq_u1d_workspace_size(const cueq_u1d_plan* plan, const cueq_u1d_buffer* buffers, int64_t batch) {
  if (!plan || !buffers) return 0;
  const int msize = plan->math_dtype == CUEQ_F64 ? 8 : 4;
  int64_t need = 0;
  for (int i = 0, n = plan_specs(plan); i < n; ++i) {
    const U1dSpec* sp = plan->specs[i].load(std::memory_order_relaxed);
    if (sp->workspace) need = std::max<int64_t>(need, sp->workspace(buffers, batch));
  }
  for (int ob = 0; ob < plan->num_outputs; ++ob) {
    const int b = plan->num_inputs + ob;
    const int64_t width = static_cast<int64_t>(plan->buffer_nseg[b]) * (plan->buffer_dim[b] ? plan->extent : 1);
    if (buffers[b].batch_dim == CUEQ_BATCH_INDEXED) {
      const int64_t splits = row_splits(batch, buffers[b].rows);
      if (splits > 1) need = std::max<int64_t>(need, splits * buffers[b].rows * width * msize);
      continue;
    }
    if (buffers[b].batch_dim != CUEQ_BATCH_SHARED) continue;
    const int64_t nch = share_chunks(batch);
    if (nch <= 1) continue;
    need = std::max<int64_t>(need, nch * width * msize);
  }
  return need;
}

// The kernels with a fixed operand count, as functors over the count.
struct RowsegPaths {
  template <typename M, int N>
  static void launch(dim3 grid, hipStream_t stream, const KernelArgs& a) {
    hipLaunchKernelGGL((u1d_rowseg_paths<M, N>), grid, dim3(256), 0, stream, a);
  }
};
struct ReducePaths {
  template <typename M, int N>
  static void launch(dim3 grid, hipStream_t stream, const KernelArgs& a) {
    hipLaunchKernelGGL((u1d_reduce_paths<M, N>), grid, dim3(256), 0, stream, a);
  }
};
template <typename M, typename K>
static void launch_by_operands(int most, dim3 grid, hipStream_t stream, const KernelArgs& a) {
  switch (most) {
    case 1: K::template launch<M, 1>(grid, stream, a); break;
    case 2: K::template launch<M, 2>(grid, stream, a); break;
    case 3: K::template launch<M, 3>(grid, stream, a); break;
    case 4: K::template launch<M, 4>(grid, stream, a); break;
    case 5: K::template launch<M, 5>(grid, stream, a); break;
    case 6: K::template launch<M, 6>(grid, stream, a); break;
    default: K::template launch<M, 7>(grid, stream, a); break;
  }
}

template <typename M>
static int run_typed(const cueq_u1d_plan* plan, const cueq_u1d_buffer* buffers, int64_t batch, void* workspace,
                     int64_t workspace_bytes, hipStream_t stream) {
  const int nbuf = plan->num_inputs + plan->num_outputs;
  KernelArgs a{};
  for (int b = 0; b < nbuf; ++b) {
    const cueq_u1d_buffer& s = buffers[b];
    CUEQ_REQUIRE(s.batch_dim == CUEQ_BATCH_SHARED || s.batch_dim == CUEQ_BATCH_BATCHED ||
                     s.batch_dim == CUEQ_BATCH_INDEXED,
                 CUEQ_ERR_INVALID, "buffer %d: batch_dim must be resolved (shared/batched/indexed)", b);
    CUEQ_REQUIRE(s.dtype >= CUEQ_F32 && s.dtype <= CUEQ_BF16, CUEQ_ERR_INVALID, "buffer %d: bad dtype", b);
    CUEQ_REQUIRE(s.rows >= 0, CUEQ_ERR_INVALID, "buffer %d: negative row count", b);
    const int64_t width = static_cast<int64_t>(plan->buffer_nseg[b]) * (plan->buffer_dim[b] ? plan->extent : 1);
    CUEQ_REQUIRE(s.data != nullptr || s.rows * width == 0, CUEQ_ERR_INVALID, "buffer %d: null data", b);
    if (s.batch_dim == CUEQ_BATCH_SHARED) CUEQ_REQUIRE(s.rows == 1, CUEQ_ERR_INVALID, "buffer %d: shared buffer must have one row", b);
    if (s.batch_dim == CUEQ_BATCH_BATCHED) CUEQ_REQUIRE(s.rows == batch, CUEQ_ERR_INVALID, "buffer %d: %lld rows, batch size is %lld", b, (long long)s.rows, (long long)batch);
    if (s.batch_dim == CUEQ_BATCH_INDEXED) {
      CUEQ_REQUIRE(s.index != nullptr || batch == 0, CUEQ_ERR_INVALID, "buffer %d: indexed without index tensor", b);
      if (b >= plan->num_inputs)
        CUEQ_REQUIRE(s.csr_offsets != nullptr && (s.csr_perm != nullptr || batch == 0), CUEQ_ERR_INVALID,
                     "output buffer %d is indexed: csr_offsets/csr_perm are required", b);
    }
    DevBuffer& dbuf = a.buf[b];
    dbuf.data = s.data;
    dbuf.index = s.index;
    dbuf.rows = s.rows;
    dbuf.dtype = s.dtype;
    dbuf.mode = s.batch_dim;
    dbuf.index_is_64 = s.index_is_64;
    dbuf.dim = plan->buffer_dim[b];
    dbuf.nseg = plan->buffer_nseg[b];
    dbuf.seg_base = plan->seg_base[b];
    dbuf.seg_stride = plan->seg_stride[b];
  }
  a.batch = batch;
  a.extent = plan->extent;
  a.chunk = kShareChunk;
  a.same_type = 1;
  for (int b = 0; b < plan->num_inputs; ++b)
    if (buffers[b].dtype != (sizeof(M) == 8 ? CUEQ_F64 : CUEQ_F32)) a.same_type = 0;

  for (int ob = 0; ob < plan->num_outputs; ++ob) {
    const int b = plan->num_inputs + ob;
    const OutTables& t = plan->out[ob];
    const cueq_u1d_buffer& o = buffers[b];
    const int ext_out = plan->buffer_dim[b] ? plan->extent : 1;
    const int64_t width = static_cast<int64_t>(plan->buffer_nseg[b]) * ext_out;
    if (o.rows * width == 0) continue;
    a.coeff = t.coeff;
    a.nin = t.nin;
    a.in = t.in;
    a.rows = t.rows;
    a.seg_start = t.seg_start;
    a.out_dim = plan->buffer_dim[b];
    a.out_nseg = plan->buffer_nseg[b];
    a.out_mode = o.batch_dim;
    a.csr_offsets = o.csr_offsets;
    a.csr_perm = o.csr_perm;
    a.out = o.data;
    a.out_dtype = o.dtype;
    a.out_rows = o.rows;
    a.out_seg_base = plan->seg_base[b];
    a.out_seg_stride = plan->seg_stride[b];
    int64_t nchunks = 0;
    a.zsplit = 1;
    a.rows_real = o.rows;
    if (o.batch_dim == CUEQ_BATCH_INDEXED && row_splits(batch, o.rows) > 1) {
      const int64_t splits = row_splits(batch, o.rows);
      const int64_t need = splits * o.rows * width * static_cast<int64_t>(sizeof(M));
      CUEQ_REQUIRE(workspace != nullptr && workspace_bytes >= need, CUEQ_ERR_INVALID, "workspace too small: need %lld bytes", (long long)need);
      a.out = workspace;
      a.out_dtype = sizeof(M) == 8 ? CUEQ_F64 : CUEQ_F32;
      a.out_rows = splits * o.rows;
      a.zsplit = static_cast<int32_t>(splits);
    }
    if (o.batch_dim == CUEQ_BATCH_SHARED) {
      nchunks = share_chunks(batch);
      if (nchunks > 1) {
        const int64_t need = nchunks * width * static_cast<int64_t>(sizeof(M));
        CUEQ_REQUIRE(workspace != nullptr && workspace_bytes >= need, CUEQ_ERR_INVALID,
                     "workspace too small: need %lld bytes", (long long)need);
        a.out = workspace;
        a.out_dtype = sizeof(M) == 8 ? CUEQ_F64 : CUEQ_F32;
        a.out_rows = nchunks;
      } else {
        a.out_rows = 1;  // zero or one chunk: fold straight into the output
      }
    }
    const bool wave = t.contracts_channel;
    const int64_t work = a.out_rows * (wave ? static_cast<int64_t>(a.out_nseg) * 64 : width);
    const int64_t blocks = (work + 255) / 256;
    CUEQ_REQUIRE(blocks < (int64_t(1) << 31), CUEQ_ERR_TOO_LARGE, "output %d too large for one launch", ob);
    // outputs that carry the channel mode (at least half a wavefront of channels): a wavefront per (row, segment, 64 channels)
    const bool rowseg = !wave && plan->buffer_dim[b] && plan->extent >= 32;
    if (rowseg) {
      const int64_t waves = a.out_rows * a.out_nseg * ((plan->extent + 63) / 64);
      const int64_t rblocks = (waves + 3) / 4;
      CUEQ_REQUIRE(rblocks < (int64_t(1) << 31), CUEQ_ERR_TOO_LARGE, "output %d too large for one launch", ob);
      const dim3 rgrid(static_cast<unsigned>(rblocks));
      if (!a.same_type) hipLaunchKernelGGL(u1d_generic_rowseg<M>, rgrid, dim3(256), 0, stream, a);
      else launch_by_operands<M, RowsegPaths>(t.max_nin, rgrid, stream, a);
    } else if (wave) {
      const dim3 wgrid(static_cast<unsigned>(blocks));
      if (!a.same_type) hipLaunchKernelGGL(u1d_generic_wave<M>, wgrid, dim3(256), 0, stream, a);
      else launch_by_operands<M, ReducePaths>(t.max_nin, wgrid, stream, a);
    }
    else hipLaunchKernelGGL(u1d_generic_elem<M>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, a);
    CUEQ_CHECK_HIP(hipGetLastError());
    if (nchunks > 1) {
      const int64_t fb = (width + 255) / 256;
      hipLaunchKernelGGL(u1d_fold_chunks<M>, dim3(static_cast<unsigned>(fb)), dim3(256), 0, stream,
                         static_cast<const M*>(workspace), nchunks, width, o.data, o.dtype);
      CUEQ_CHECK_HIP(hipGetLastError());
    }
    if (a.zsplit > 1) {  // the pieces of every row, added in order
      const int64_t elems = o.rows * width, fb = (elems + 255) / 256;
      CUEQ_REQUIRE(fb < (int64_t(1) << 31), CUEQ_ERR_TOO_LARGE, "output %d too large for one launch", ob);
      hipLaunchKernelGGL(u1d_fold_chunks<M>, dim3(static_cast<unsigned>(fb)), dim3(256), 0, stream,
                         static_cast<const M*>(workspace), static_cast<int64_t>(a.zsplit), elems, o.data, o.dtype);
      CUEQ_CHECK_HIP(hipGetLastError());
    }
  }
  return CUEQ_OK;
}

extern "C" int cueq_u1d_run(const cueq_u1d_plan* plan, const cueq_u1d_buffer* buffers, int64_t batch, void* workspace,
                            int64_t workspace_bytes, void* stream) {
  CUEQ_REQUIRE(plan && buffers, CUEQ_ERR_INVALID, "null argument");
  CUEQ_REQUIRE(batch >= 0, CUEQ_ERR_INVALID, "negative batch size");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (!opt_force_generic().load(std::memory_order_relaxed)) {
    SpecCall call{buffers, batch, workspace, workspace_bytes, s};
    for (int i = 0, n = plan_specs(plan); i < n; ++i) {
      const int rc = plan->specs[i].load(std::memory_order_relaxed)->run(call);
      if (rc != CUEQ_ERR_UNSUPPORTED) return rc;
    }
  }
  if (plan->math_dtype == CUEQ_F64) return run_typed<double>(plan, buffers, batch, workspace, workspace_bytes, s);
  return run_typed<float>(plan, buffers, batch, workspace, workspace_bytes, s);
}

// ---- cueq_u1d_run for callers that cannot allocate -------------------------------------------------
// The workspace of cueq_u1d_run (per-chunk partial rows of a batch-reduced output, per-channel-half partials of the
// fused backward) lives in a file-scope device array instead of a caller-supplied buffer.  Every device that loads
// this library holds its own copy of the array until the process ends.  The array's name is only a host-side handle:
// the address a kernel may use is asked for once per device with hipGetSymbolAddress and kept.
namespace cueq {
constexpr int64_t kStaticScratchBytes = int64_t(32) << 20;  // 32 MiB
constexpr int kMaxScratchDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static void* g_scratch_ptr[kMaxScratchDevices] = {};
static std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device (looked up on the first call on that device).
static int static_scratch(void** out) {
  int dev = 0;
  CUEQ_CHECK_HIP(hipGetDevice(&dev));
  CUEQ_REQUIRE(dev >= 0 && dev < kMaxScratchDevices, CUEQ_ERR_UNSUPPORTED, "device %d beyond the %d this entry point serves", dev,
               kMaxScratchDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    CUEQ_CHECK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    CUEQ_REQUIRE(p != nullptr, CUEQ_ERR_HIP, "hipGetSymbolAddress returned a null address for the static scratch array");
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return CUEQ_OK;
}
}  // namespace cueq

extern "C" int64_t cueq_u1d_static_scratch_bytes(void) { return cueq::kStaticScratchBytes; }

extern "C" int cueq_u1d_run_static(const cueq_u1d_plan* plan, const cueq_u1d_buffer* buffers, int64_t batch, void* stream) {
  CUEQ_REQUIRE(plan && buffers, CUEQ_ERR_INVALID, "null argument");
  CUEQ_REQUIRE(batch >= 0, CUEQ_ERR_INVALID, "negative batch size");
  const int64_t need = cueq_u1d_workspace_size(plan, buffers, batch);
  CUEQ_REQUIRE(need <= cueq::kStaticScratchBytes, CUEQ_ERR_TOO_LARGE,
               "this call needs %lld bytes of scratch, the static array holds %lld: use cueq_u1d_run with a workspace",
               (long long)need, (long long)cueq::kStaticScratchBytes);
  void* ws = nullptr;
  if (need > 0) {
    const int rc = cueq::static_scratch(&ws);
    if (rc != CUEQ_OK) return rc;
  }
  // Every kernel that uses the workspace writes each element it later reads (partial rows are stored, not
  // accumulated), so nothing has to be cleared between calls.
  return cueq_u1d_run(plan, buffers, batch, ws, need > 0 ? cueq::kStaticScratchBytes : 0, stream);
}
