// Registry of descriptor-specialised uniform-1d kernels.
//
// The generic executor interprets path tables at run time.  For descriptors known when the
// library is built, straight-line kernels are generated (cuequivariance_amd/codegen) with the
// path table baked into the instruction stream; each generated translation unit registers
// itself here under a content hash of the descriptor tables.  cueq_u1d_plan_create computes the
// same hash and, when it finds entries, cueq_u1d_run tries them first; an entry may decline a
// call shape (returns CUEQ_ERR_UNSUPPORTED), in which case the generic kernels run.  One descriptor may have several
// entries: one per element type of the buffers (the arithmetic type itself, and 16-bit elements for float arithmetic).
#pragma once

#include <cstdint>

#include "common.h"

namespace cueq {

struct SpecCall {
  const cueq_u1d_buffer* buffers;  // inputs then outputs
  int64_t batch;
  void* workspace;
  int64_t workspace_bytes;
  hipStream_t stream;
};

struct U1dSpec {
  uint64_t hash;
  const char* name;
  int (*run)(const SpecCall& call);                                    // CUEQ_OK / CUEQ_ERR_UNSUPPORTED / error
  int64_t (*workspace)(const cueq_u1d_buffer* buffers, int64_t batch);  // bytes, may be null
  int io_dtype;  // CUEQ_* code of the buffers this entry takes (all buffers of a call hold the same type)
};

void register_u1d_spec(const U1dSpec* spec);
// the entry for `hash` whose buffers hold `io_dtype`; io_dtype < 0: the one whose buffers hold the arithmetic type
const U1dSpec* find_u1d_spec(uint64_t hash, int io_dtype = -1);

// FNV-1a over a stream of 64-bit words (little endian bytes); the generator computes the same.
struct Fnv64 {
  uint64_t h = 1469598103934665603ull;
  void word(uint64_t w) {
    for (int i = 0; i < 8; ++i) {
      h ^= (w >> (8 * i)) & 0xff;
      h *= 1099511628211ull;
    }
  }
};

uint64_t hash_u1d_desc(const cueq_u1d_desc* d);

// Optional per-kernel timing with HIP events (cueq_timing_begin / cueq_timing_end).
bool timing_enabled();
void timing_mark(const char* name, hipStream_t stream, bool begin);

struct KernelTimer {
  const char* name;
  hipStream_t stream;
  bool on;
  KernelTimer(const char* n, hipStream_t s) : name(n), stream(s), on(timing_enabled()) {
    if (on) timing_mark(name, stream, true);
  }
  ~KernelTimer() {
    if (on) timing_mark(name, stream, false);
  }
};

struct SpecRegistrar {
  explicit SpecRegistrar(const U1dSpec* s) { register_u1d_spec(s); }
};

}  // namespace cueq
