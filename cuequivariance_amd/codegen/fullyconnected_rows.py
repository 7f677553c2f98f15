"""Kernels for a fully connected tensor product whose weights differ from batch row to batch row (``uvw,iu,jv,kw+ijk`` with
``v = 1``, weights of shape ``(batch, weight_numel)``): the product inside
``cuequivariance_torch/layers/tp_conv_fully_connected.py:216-276`` (an MLP makes the weights of every edge), which the
reference runs through ``FullyConnectedTensorProduct`` with ``shared_weights=False``
(``cuequivariance_torch/operations/tp_fully_connected.py:30-207``).

Every weight is used for ``2 (2 l3 + 1)`` flops and read once: the product streams the weights (20 480 values per edge for
``64x0e+64x1o (x) 0e+1o+2e -> 64x0e+64x1o``), there is nothing for the matrix cores to reuse.  One wavefront works on one
batch row at a time.  With ``S_p[k, u] = sum_ij C_p[i, j, k] x1[i, u] x2[j]`` (a lane per ``u``):

* forward (a wavefront per output row, its batch rows in order - bit-reproducible):
  ``out[k, w] += sum_u W_p[u, w] S_p[k, u]``, a lane per ``w``, ``S_p[k, u]`` read from lane ``u``;
* backward, all three gradients in one pass over the weights (a wavefront per range of batch rows):
  ``dW_p[u, w] = sum_k S_p[k, u] g[k, w]`` (a lane per ``w``, stored as the weight row was loaded), and with
  ``R_p[k, u] = sum_w W_p[u, w] g[k, w]`` - the weight block goes through LDS once and is read back by columns, a lane
  per ``u`` - ``dx1[i, u] += sum_jk C_p[i, j, k] x2[j] R_p[k, u]`` and ``dx2[j] += sum_u sum_ik C_p[i, j, k] x1[i, u] R_p[k, u]``.

The unit registers under the hashes of the flattened uniform-1d tables (forward, and backward for all three inputs), like
the channel-wise units; buffers and batch modes are those of ``codegen/channelwise.py``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Tuple


MAX_GROUP = 16


@dataclass
class Block:
    w_off: int          # element offset of the (U x Wd) weight block in a weight row
    a_off: int          # element offset of the x1 segment (d1 x U)
    d1: int
    b_off: int          # element offset of the x2 segment (d2)
    d2: int
    c_off: int          # element offset of the output segment (d3 x Wd)
    d3: int
    entries: List[Tuple[int, int, int, float]] = field(default_factory=list)  # (i, j, k, coefficient), non-zero


@dataclass
class RowWeightStructure:
    U: int
    Wd: int
    width_w: int
    width_x1: int
    width_x2: int
    width_out: int
    blocks: List[Block]


def analyze(polynomial) -> Optional[RowWeightStructure]:
    """The structure of ``uvw,iu,jv,kw+ijk`` with ``v = 1`` and one multiplicity per operand (at most 64), else None."""
    if polynomial is None or polynomial.num_inputs != 3 or polynomial.num_outputs != 1 or len(polynomial.operations) != 1:
        return None
    ope, stp = polynomial.operations[0]
    if tuple(ope.buffers) != (0, 1, 2, 3) or str(stp.subscripts) != "uvw,iu,jv,kw+ijk":
        return None
    ow, o1, o2, oo = stp.operands
    if not o1.segments or not oo.segments or not stp.paths:
        return None
    U, Wd = o1.segments[0][1], oo.segments[0][1]
    if any(s[1] != U for s in o1.segments) or any(s[1] != Wd for s in oo.segments) or any(s[1] != 1 for s in o2.segments):
        return None
    if any(tuple(s) != (U, 1, Wd) for s in ow.segments) or U > 64 or Wd > 64:
        return None

    def offsets(operand):
        out, off = [], 0
        for s in operand.segments:
            out.append(off)
            n = 1
            for e in s:
                n *= e
            off += n
        return out, off

    offw, nw = offsets(ow)
    off1, n1 = offsets(o1)
    off2, n2 = offsets(o2)
    offo, no = offsets(oo)
    blocks = []
    for path in stp.paths:
        sw, s1, s2, so = path.indices
        blk = Block(offw[sw], off1[s1], o1.segments[s1][0], off2[s2], o2.segments[s2][0], offo[so], oo.segments[so][0])
        c = path.coefficients
        for i in range(blk.d1):
            for j in range(blk.d2):
                for k in range(blk.d3):
                    if c[i, j, k] != 0:
                        blk.entries.append((i, j, k, float(c[i, j, k])))
        if blk.entries:
            blocks.append(blk)
    if not blocks:
        return None
    return RowWeightStructure(U, Wd, nw, n1, n2, no, blocks)


def _lit(c: float, T: str) -> str:
    return f"{c!r}" + ("f" if T == "float" else "")


def _s_terms(st: RowWeightStructure, blk: Block, T: str, x1: str, x2: str):
    """{k: expression of S[k] = sum_ij c x1[i] x2[j]} for one block (per-lane values, a lane per u)."""
    by_k = {}
    for i, j, k, c in blk.entries:
        term = f"{_lit(c, T)} * {x1}{(blk.a_off // st.U) + i} * {x2}{blk.b_off + j}"
        by_k.setdefault(k, []).append(term)
    return {k: " + ".join(v) for k, v in by_k.items()}


def emit_unit(st: RowWeightStructure, T: str, name: str, fwd_hash: int, bwd_hash: int) -> str:
    U, Wd = st.U, st.Wd
    nx1 = st.width_x1 // U          # x1 components (each a vector over u)
    nout = st.width_out // Wd       # output components (each a vector over w)
    n2 = st.width_x2
    TS = 65                         # row stride of the LDS tile in elements: column reads touch every bank once
    G = next(n for n in (32, 16, 8, 4, 2, 1) if n <= MAX_GROUP and U % n == 0)  # weight rows requested together, one group ahead of their use
    waves = 2 if T == "float" else 1
    L: List[str] = []
    A = L.append
    A("// GENERATED by cuequivariance_amd/codegen/fullyconnected_rows.py - do not edit.")
    A(f"// fully connected product with a weight row per batch row '{name}': U = {U}, W = {Wd}, {len(st.blocks)} blocks, "
      f"widths w/x1/x2/out = {st.width_w}/{st.width_x1}/{st.width_x2}/{st.width_out}, math {T}")
    A('#include "cw_common.h"')
    A("#define STREAM_LOAD(p) __builtin_nontemporal_load(p)")
    A("#define STREAM_STORE(v, p) __builtin_nontemporal_store(v, p)")
    A("")
    A("namespace cueq {")
    A(f"namespace fcr_{name} {{")
    A("")
    A("// the value lane `src` (the same for every lane) holds")
    A("__device__ __forceinline__ float lane_value(float v, int src) { return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), src)); }")
    A("__device__ __forceinline__ double lane_value(double v, int src) {")
    A("  const uint64_t b = __builtin_bit_cast(uint64_t, v);")
    A("  const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(b & 0xffffffffu), src));")
    A("  const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(b >> 32), src));")
    A("  return __builtin_bit_cast(double, (static_cast<uint64_t>(hi) << 32) | lo);")
    A("}")
    A("")

    # ------------------------------------------------------------------ forward
    A("// forward: `parts` wavefronts per output row, each sums a contiguous piece of the row's batch rows in list order (one")
    A("// wavefront per row when there are enough rows to fill the chip; else the pieces go to partial rows, folded in order)")
    A("template <bool X1_IDX>")
    A(f"__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu({waves}))) fwd_kernel(")
    A(f"    const {T}* __restrict__ w, const {T}* __restrict__ x1, const {T}* __restrict__ x2, {T}* __restrict__ out,")
    A("    const void* __restrict__ x1_index, int x1_idx64, const int64_t* __restrict__ csr_offsets, const int64_t* __restrict__ csr_perm, int parts) {")
    A("  const int lane = threadIdx.x;")
    A("  const int64_t r = blockIdx.x / parts;")
    A("  const int part = static_cast<int>(blockIdx.x - r * parts);")
    A(f"  const bool act_u = lane < {U}, act_w = lane < {Wd};")
    A(f"  const int lu = act_u ? lane : 0, lw = act_w ? lane : 0;")
    for k in range(nout):
        A(f"  {T} acc{k} = 0;")
    A("  int64_t z0, z1;")
    A("  if (csr_offsets) { z0 = csr_offsets[r]; z1 = csr_offsets[r + 1]; } else { z0 = r; z1 = r + 1; }")
    A("  { const int64_t n = z1 - z0; z1 = z0 + n * (part + 1) / parts; z0 = z0 + n * part / parts; }")
    A("  for (int64_t zz = z0; zz < z1; ++zz) {")
    A("    const int64_t z = csr_perm ? csr_perm[zz] : zz;")
    A("    int64_t srow = z;")
    A("    if (X1_IDX) srow = x1_idx64 ? static_cast<const int64_t*>(x1_index)[z] : static_cast<int64_t>(static_cast<const int32_t*>(x1_index)[z]);")
    A(f"    const {T}* __restrict__ x1p = x1 + srow * {st.width_x1}ll;")
    A(f"    const {T}* __restrict__ x2p = x2 + z * {n2}ll;")
    A(f"    const {T}* __restrict__ wp = w + z * {st.width_w}ll + lw;")
    for i in range(nx1):
        A(f"    const {T} xa{i} = act_u ? x1p[{i * U} + lu] : {T}(0);")
    for j in range(n2):
        A(f"    const {T} xb{j} = x2p[{j}];")
    groups = [(b, g0) for b, blk in enumerate(st.blocks) for g0 in range(0, U, G)]

    def load_group(ind: str, which: int, b: int, g0: int, guard: str = ""):
        for r in range(G):
            A(f"{ind}wq{which}_{r} = {guard}STREAM_LOAD(wp + {st.blocks[b].w_off} + {(g0 + r) * Wd});")

    A(f"    {T} " + ", ".join(f"wq{q}_{r}" for q in range(2) for r in range(G)) + ";")
    load_group("    ", 0, *groups[0])
    for gi, (b, g0) in enumerate(groups):
        blk = st.blocks[b]
        if g0 == 0:
            S = _s_terms(st, blk, T, "xa", "xb")
            A(f"    // block {b}: x1 segment at {blk.a_off}, x2 at {blk.b_off}, output at {blk.c_off}")
            for k, e in sorted(S.items()):
                A(f"    const {T} S{b}_{k} = {e};")
        if gi + 1 < len(groups):
            load_group("    ", (gi + 1) & 1, *groups[gi + 1])
        for r in range(G):
            for k in sorted(S):
                A(f"    acc{blk.c_off // Wd + k} = fma(wq{gi & 1}_{r}, lane_value(S{b}_{k}, {g0 + r}), acc{blk.c_off // Wd + k});")
    A("  }")
    A(f"  {T}* __restrict__ op = out + static_cast<int64_t>(blockIdx.x) * {st.width_out}ll + lw;  // (out = the partial rows when parts > 1)")
    A("  if (act_w) {")
    for k in range(nout):
        A(f"    STREAM_STORE(acc{k}, op + {k * Wd});")
    A("  }")
    A("}")
    A("")

    # ------------------------------------------------------------------ backward
    A("// backward: dw, dx1, dx2 in one pass over the weights; every wavefront owns one contiguous range of batch rows")
    A("template <bool X1_IDX, bool G_IDX, bool ATOMIC_DX1>")
    A(f"__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu({waves}))) bwd_kernel(")
    A(f"    const {T}* __restrict__ w, const {T}* __restrict__ x1, const {T}* __restrict__ x2, const {T}* __restrict__ g,")
    A(f"    {T}* __restrict__ dw, {T}* dx1, {T}* __restrict__ dx1_partial, {T}* __restrict__ dx2,")
    A("    const void* __restrict__ x1_index, int x1_idx64, const void* __restrict__ g_index, int g_idx64, int64_t batch) {")
    A(f"  __shared__ {T} tile[{64 * TS}];  // one weight block: row u at u * {TS}")
    A("  const int lane = threadIdx.x;")
    A(f"  const bool act_u = lane < {U}, act_w = lane < {Wd};")
    A("  const int lu = act_u ? lane : 0, lw = act_w ? lane : 0;")
    A("  const int64_t z0 = blockIdx.x * batch / gridDim.x, z1 = (blockIdx.x + 1) * batch / gridDim.x;")
    A("  for (int64_t z = z0; z < z1; ++z) {")
    A("    int64_t srow = z, grow = z;")
    A("    if (X1_IDX) srow = x1_idx64 ? static_cast<const int64_t*>(x1_index)[z] : static_cast<int64_t>(static_cast<const int32_t*>(x1_index)[z]);")
    A("    if (G_IDX) grow = g_idx64 ? static_cast<const int64_t*>(g_index)[z] : static_cast<int64_t>(static_cast<const int32_t*>(g_index)[z]);")
    A(f"    const {T}* __restrict__ x1p = x1 + srow * {st.width_x1}ll;")
    A(f"    const {T}* __restrict__ x2p = x2 + z * {n2}ll;")
    A(f"    const {T}* __restrict__ gp = g + grow * {st.width_out}ll;")
    A(f"    const {T}* __restrict__ wp = w + z * {st.width_w}ll + lw;")
    A(f"    {T}* __restrict__ dwp = dw + z * {st.width_w}ll + lw;")
    for i in range(nx1):
        A(f"    const {T} xa{i} = act_u ? x1p[{i * U} + lu] : {T}(0);")
    for j in range(n2):
        A(f"    const {T} xb{j} = x2p[{j}];")
    for k in range(nout):
        A(f"    const {T} gv{k} = act_w ? gp[{k * Wd} + lw] : {T}(0);")
    for i in range(nx1):
        A(f"    {T} da{i} = 0;")
    for j in range(n2):
        A(f"    {T} db{j} = 0;")
    zero = f"{T}(0)"
    A(f"    {T} " + ", ".join(f"wq{q}_{r}" for q in range(2) for r in range(G)) + ";")

    def load_group_b(ind: str, which: int, b: int, g0: int):
        for r in range(G):
            A(f"{ind}wq{which}_{r} = act_w ? STREAM_LOAD(wp + {st.blocks[b].w_off} + {(g0 + r) * Wd}) : {zero};")

    load_group_b("    ", 0, *groups[0])
    for gi, (b, g0) in enumerate(groups):
        blk = st.blocks[b]
        kb = blk.c_off // Wd
        if g0 == 0:
            S = _s_terms(st, blk, T, "xa", "xb")
            ks = sorted(S)
            A(f"    // block {b}")
            for k, e in sorted(S.items()):
                A(f"    const {T} S{b}_{k} = {e};")
        if gi + 1 < len(groups):
            load_group_b("    ", (gi + 1) & 1, *groups[gi + 1])
        for r in range(G):
            u = g0 + r
            A(f"    tile[{u * TS} + lane] = wq{gi & 1}_{r};")
            expr = None
            for k in ks:
                expr = f"lane_value(S{b}_{k}, {u}) * gv{kb + k}" if expr is None else f"fma(lane_value(S{b}_{k}, {u}), gv{kb + k}, {expr})"
            A(f"    if (act_w) STREAM_STORE({expr}, dwp + {blk.w_off} + {u * Wd});")
        if g0 + G >= U:  # the block is complete in LDS: read it back by columns, a lane per u
            A("    __builtin_amdgcn_fence(__ATOMIC_RELEASE, \"wavefront\");")
            A("    __builtin_amdgcn_wave_barrier();")
            A("    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, \"wavefront\");")
            A("    {")
            for k in ks:
                A(f"      {T} R{k} = 0;")
            A("#pragma unroll 16")
            A(f"      for (int c = 0; c < {Wd}; ++c) {{")
            A(f"        const {T} wc = tile[lu * {TS} + c];")
            for k in ks:
                A(f"        R{k} = fma(wc, lane_value(gv{kb + k}, c), R{k});")
            A("      }")
            for i, j, k, c in blk.entries:
                ai = blk.a_off // U + i
                A(f"      da{ai} = fma({_lit(c, T)} * xb{blk.b_off + j}, R{k}, da{ai}); db{blk.b_off + j} = fma({_lit(c, T)} * xa{ai}, R{k}, db{blk.b_off + j});")
            A("    }")
            A("    __builtin_amdgcn_fence(__ATOMIC_RELEASE, \"wavefront\");")
            A("    __builtin_amdgcn_wave_barrier();")
            A("    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, \"wavefront\");")
    # gradients of the row
    A("    if (act_u) {")
    A("      if (ATOMIC_DX1) {")
    A(f"        {T}* dp = dx1 + srow * {st.width_x1}ll + lu;")
    for i in range(nx1):
        A(f"        unsafeAtomicAdd(dp + {i * U}, da{i});")
    A("      } else {")
    A(f"        {T}* __restrict__ dp = dx1_partial + z * {st.width_x1}ll + lu;")
    for i in range(nx1):
        A(f"        dp[{i * U}] = da{i};")
    A("      }")
    A("    }")
    for j in range(n2):
        A(f"    db{j} = wave_sum(act_u ? db{j} : {T}(0));")
    A("    if (lane == 0) {")
    A(f"      {T}* __restrict__ d2 = dx2 + z * {n2}ll;")
    for j in range(n2):
        A(f"      d2[{j}] = db{j};")
    A("    }")
    A("  }")
    A("}")
    A("")
    code = f"dtype_code<{T}>::value"
    W1 = st.width_x1
    A(f"""
static bool all_dtype(const cueq_u1d_buffer* b, int n) {{
  for (int i = 0; i < n; ++i) if (b[i].dtype != {code}) return false;
  return true;
}}

// buffers: w, x1, x2 | out
// wavefronts per output row: one when the rows fill the chip about three times over, else up to 8 pieces per row - but
// no more pieces than a row has batch rows on average
static int fwd_parts(const cueq_u1d_buffer* b, int64_t batch) {{
  if (b[3].batch_dim != CUEQ_BATCH_INDEXED || b[3].rows <= 0) return 1;
  const int64_t want = (3 * wave_slots({waves}) + b[3].rows - 1) / b[3].rows, mean = batch / b[3].rows;
  int64_t p = want < mean ? want : mean;
  if (p > 8) p = 8;
  return p < 1 ? 1 : static_cast<int>(p);
}}
static int64_t fwd_workspace(const cueq_u1d_buffer* b, int64_t batch) {{
  const int parts = fwd_parts(b, batch);
  return parts > 1 ? b[3].rows * parts * {st.width_out}ll * sizeof({T}) : 0;
}}

static int run_fwd(const SpecCall& c) {{
  const cueq_u1d_buffer* b = c.buffers;
  if (!all_dtype(b, 4)) return CUEQ_ERR_UNSUPPORTED;
  if (b[0].batch_dim != CUEQ_BATCH_BATCHED || b[2].batch_dim != CUEQ_BATCH_BATCHED) return CUEQ_ERR_UNSUPPORTED;
  if (b[1].batch_dim == CUEQ_BATCH_SHARED || b[3].batch_dim == CUEQ_BATCH_SHARED) return CUEQ_ERR_UNSUPPORTED;
  const bool x1_idx = b[1].batch_dim == CUEQ_BATCH_INDEXED, out_idx = b[3].batch_dim == CUEQ_BATCH_INDEXED;
  if (out_idx && (!b[3].csr_offsets || (!b[3].csr_perm && c.batch > 0))) return CUEQ_ERR_UNSUPPORTED;
  const int64_t rows = b[3].rows;
  if (rows == 0) return CUEQ_OK;
  const int parts = fwd_parts(b, c.batch);
  CUEQ_REQUIRE(rows * parts < (int64_t(1) << 31), CUEQ_ERR_TOO_LARGE, "too many output rows for one launch");
  const int64_t need = fwd_workspace(b, c.batch);
  CUEQ_REQUIRE(need == 0 || (c.workspace && c.workspace_bytes >= need), CUEQ_ERR_INVALID, "workspace too small: need %lld bytes", (long long)need);
  const {T}* w = static_cast<const {T}*>(b[0].data);
  const {T}* x1 = static_cast<const {T}*>(b[1].data);
  const {T}* x2 = static_cast<const {T}*>(b[2].data);
  {T}* o = static_cast<{T}*>(b[3].data);
  const int64_t* offs = out_idx ? b[3].csr_offsets : nullptr;
  const int64_t* perm = out_idx ? b[3].csr_perm : nullptr;
  const dim3 g(static_cast<unsigned>(rows * parts)), t(64);
  {T}* dst = parts > 1 ? static_cast<{T}*>(c.workspace) : o;
  {{
    KernelTimer timer("{name}_fwd_{T}", c.stream);
    if (x1_idx) hipLaunchKernelGGL((fwd_kernel<true>), g, t, 0, c.stream, w, x1, x2, dst, b[1].index, b[1].index_is_64, offs, perm, parts);
    else hipLaunchKernelGGL((fwd_kernel<false>), g, t, 0, c.stream, w, x1, x2, dst, b[1].index, b[1].index_is_64, offs, perm, parts);
  }}
  CUEQ_CHECK_HIP(hipGetLastError());
  if (parts > 1) {{
    hipLaunchKernelGGL(fold_parts<{T}>, dim3(blocks_for(rows * {st.width_out}ll)), dim3(256), 0, c.stream, dst, rows, parts, {st.width_out}, o);
    CUEQ_CHECK_HIP(hipGetLastError());
  }}
  return CUEQ_OK;
}}

// buffers: w, x1, x2, g | dw, dx1, dx2
static int64_t bwd_workspace(const cueq_u1d_buffer* b, int64_t batch) {{
  if (b[1].batch_dim == CUEQ_BATCH_INDEXED && deterministic_scatter()) return batch * {W1}ll * sizeof({T});
  return 0;
}}

static int run_bwd(const SpecCall& c) {{
  const cueq_u1d_buffer* b = c.buffers;
  if (!all_dtype(b, 7)) return CUEQ_ERR_UNSUPPORTED;
  if (b[0].batch_dim != CUEQ_BATCH_BATCHED || b[2].batch_dim != CUEQ_BATCH_BATCHED) return CUEQ_ERR_UNSUPPORTED;
  if (b[1].batch_dim == CUEQ_BATCH_SHARED || b[3].batch_dim == CUEQ_BATCH_SHARED) return CUEQ_ERR_UNSUPPORTED;
  if (b[4].batch_dim != CUEQ_BATCH_BATCHED || b[6].batch_dim != CUEQ_BATCH_BATCHED) return CUEQ_ERR_UNSUPPORTED;
  if (b[5].batch_dim != b[1].batch_dim) return CUEQ_ERR_UNSUPPORTED;
  const bool x1_idx = b[1].batch_dim == CUEQ_BATCH_INDEXED, g_idx = b[3].batch_dim == CUEQ_BATCH_INDEXED;
  if (x1_idx && (b[5].index != b[1].index || b[5].rows != b[1].rows)) return CUEQ_ERR_UNSUPPORTED;
  const bool det = deterministic_scatter();
  if (x1_idx && det && (!b[5].csr_offsets || (!b[5].csr_perm && c.batch > 0))) return CUEQ_ERR_UNSUPPORTED;
  const int64_t batch = c.batch;
  const {T}* w = static_cast<const {T}*>(b[0].data);
  const {T}* x1 = static_cast<const {T}*>(b[1].data);
  const {T}* x2 = static_cast<const {T}*>(b[2].data);
  const {T}* g = static_cast<const {T}*>(b[3].data);
  {T}* dw = static_cast<{T}*>(b[4].data);
  {T}* dx1 = static_cast<{T}*>(b[5].data);
  {T}* dx2 = static_cast<{T}*>(b[6].data);
  const int64_t need = bwd_workspace(b, batch);
  CUEQ_REQUIRE(need == 0 || (c.workspace && c.workspace_bytes >= need), CUEQ_ERR_INVALID, "workspace too small: need %lld bytes", (long long)need);
  {T}* dx1_partial = nullptr;
  bool atomic = false;
  if (!x1_idx) dx1_partial = dx1;  // one row per batch element: plain stores
  else if (det) dx1_partial = static_cast<{T}*>(c.workspace);
  else atomic = true;
  if (atomic && b[5].rows > 0) {{
    const int64_t n = b[5].rows * {W1}ll;
    hipLaunchKernelGGL(fill_zero<{T}>, dim3(fill_blocks<{T}>(n)), dim3(256), 0, c.stream, dx1, n);
    CUEQ_CHECK_HIP(hipGetLastError());
  }}
  if (batch > 0) {{
    // one round of resident wavefronts (the LDS tile bounds them at {8 if T == "float" else 4} per CU); short batches get fewer
    int64_t nranges = static_cast<int64_t>(device_cus()) * {8 if T == "float" else 4};
    if (nranges > batch) nranges = batch;
    const dim3 gd(static_cast<unsigned>(nranges)), t(64);
    KernelTimer timer("{name}_bwd_{T}", c.stream);
#define LAUNCH_BWD(XI, GI, AT) hipLaunchKernelGGL((bwd_kernel<XI, GI, AT>), gd, t, 0, c.stream, w, x1, x2, g, dw, dx1, dx1_partial, dx2, b[1].index, b[1].index_is_64, b[3].index, b[3].index_is_64, batch)
    if (x1_idx && g_idx && atomic) LAUNCH_BWD(true, true, true);
    else if (x1_idx && g_idx) LAUNCH_BWD(true, true, false);
    else if (x1_idx && atomic) LAUNCH_BWD(true, false, true);
    else if (x1_idx) LAUNCH_BWD(true, false, false);
    else if (g_idx) LAUNCH_BWD(false, true, false);
    else LAUNCH_BWD(false, false, false);
#undef LAUNCH_BWD
    CUEQ_CHECK_HIP(hipGetLastError());
  }}
  if (x1_idx && det && b[5].rows > 0) {{
    const int64_t n = b[5].rows * {W1}ll;
    if ({W1} % 4 == 0 && reinterpret_cast<uintptr_t>(dx1) % (4 * sizeof({T})) == 0 && reinterpret_cast<uintptr_t>(dx1_partial) % (4 * sizeof({T})) == 0 &&
        b[5].rows < 65536) {{
      hipLaunchKernelGGL(segment_sum_rows_vec<{T}>, dim3(({W1} / 4 + 255) / 256, static_cast<unsigned>(b[5].rows)), dim3(256), 0, c.stream,
                         dx1_partial, b[5].csr_offsets, b[5].csr_perm, {W1}, dx1);
    }} else {{
      hipLaunchKernelGGL(segment_sum_rows<{T}>, dim3(blocks_for(n)), dim3(256), 0, c.stream, dx1_partial, b[5].csr_offsets, b[5].csr_perm, b[5].rows, {W1}, dx1);
    }}
    CUEQ_CHECK_HIP(hipGetLastError());
  }}
  return CUEQ_OK;
}}

static const U1dSpec spec_fwd = {{0x{fwd_hash:016x}ull, "{name}_fwd_{T}", run_fwd, fwd_workspace, {code}}};
static const U1dSpec spec_bwd = {{0x{bwd_hash:016x}ull, "{name}_bwd_{T}", run_bwd, bwd_workspace, {code}}};
static SpecRegistrar reg_fwd(&spec_fwd);
static SpecRegistrar reg_bwd(&spec_bwd);
""")
    A(f"}}  // namespace fcr_{name}")
    A("}  // namespace cueq")
    return "\n".join(L) + "\n"
