"""Generator of straight-line gfx950 kernels for weighted channel-wise tensor products.

Input: the flat uniform-1d tables of one operation with operands
``[w (u-vector), x1 (u-vector), x2 (scalar), out (u-vector)]`` — the form a channel-wise
tensor product takes after flattening the Clebsch-Gordan modes — i.e. for every path ``p``

    out[k_p, u] += c_p * w[b_p, u] * x1[i_p, u] * x2[j_p]

Output: HIP source with the path table unrolled into the instruction stream.

Forward kernel (one wavefront = one output row x 64 channels):
  * channels across lanes, so every HBM access is a contiguous 256-byte (fp32) line;
  * the uniform factor ``c_p * x2[j_p]`` of each path lives in a table register: lane ``n`` of each
    16-lane row holds the factor of a path whose ``x2`` index is ``n``; the FMA reads it with the DPP
    ``row_newbcast:n`` modifier, which broadcasts lane ``n`` of every row to the row - no LDS traffic,
    no scalar float arithmetic, one VALU instruction per path;
  * ``w[b] * x1[i]`` is formed once per (block, i) and reused by all paths of the block;
  * the batch rows that scatter into one output row are summed in registers in CSR order, then
    stored once: deterministic, nothing of batch size is materialised.

Backward kernel (one wavefront per resident slot, each owning a contiguous range of batch rows x 64
channels) computes the three gradients in one pass over the inputs.  With ``G[b][i][j] = sum_k C[i,j,k] g[k]`` (literal
coefficients), ``D[b][i] = sum_j G[b][i][j] x2[j]`` and ``F[b][j] = sum_i G[b][i][j] x1[i]``:
``dw[b] = sum_i x1[i] D[b][i]``, ``dx1[i] += w[b] D[b][i]``, ``dx2[j] = sum_u w[b] F[b][j]``.
"""

from __future__ import annotations

import struct
from collections import defaultdict
from dataclasses import dataclass, field
from typing import Sequence

MASK64 = (1 << 64) - 1


# ---------------------------------------------------------------------------------------------
# descriptor hash (must match cueq::hash_u1d_desc in csrc/uniform1d.hip)
# ---------------------------------------------------------------------------------------------
def fnv64_words(words) -> int:
    h = 1469598103934665603
    for w in words:
        w &= MASK64
        for i in range(8):
            h ^= (w >> (8 * i)) & 0xFF
            h = (h * 1099511628211) & MASK64
    return h


def hash_tables(math_code: int, extent: int, nin: int, nout: int, buffer_dim, nseg, num_operands, operations,
                num_paths, path_indices_start, path_coefficients_start, path_indices, path_coefficients) -> int:
    words = [math_code, extent, nin, nout, *buffer_dim, *nseg, len(num_operands)]
    off = 0
    for o, nop in enumerate(num_operands):
        words.append(nop)
        words += list(operations[off: off + nop])
        off += nop
        words.append(num_paths[o])
        pi0, pc0 = path_indices_start[o], path_coefficients_start[o]
        words += list(path_indices[pi0: pi0 + num_paths[o] * nop])
        for p in range(num_paths[o]):
            words.append(struct.unpack("<Q", struct.pack("<d", float(path_coefficients[pc0 + p])))[0])
    return fnv64_words(words)


# ---------------------------------------------------------------------------------------------
# structure analysis
# ---------------------------------------------------------------------------------------------
@dataclass
class Block:
    """All paths sharing one weight segment."""

    b: int
    entries: list = field(default_factory=list)  # (i, j, k, c)

    @property
    def i_list(self):
        return sorted({e[0] for e in self.entries})

    @property
    def j_list(self):
        return sorted({e[1] for e in self.entries})

    @property
    def k_list(self):
        return sorted({e[2] for e in self.entries})


@dataclass
class ChannelwiseStructure:
    extent: int
    nseg_w: int
    nseg_x1: int
    nseg_x2: int
    nseg_out: int
    blocks: list
    # row layouts of x1 (also of its gradient) and of the output (also of its cotangent): () = segment s, channel u at
    # s * extent + u; group sizes (d_0, d_1, ...) = groups of consecutive segments stored channel-major ("mul_ir")
    layout_x1: tuple = ()
    layout_out: tuple = ()
    # x2 = spherical harmonics of a 3-vector, evaluated in the kernels: per x2 segment its terms
    # ((sorted indices into the vector, coefficient), ...); () = x2 is read from memory
    harmonics: tuple = ()

    @property
    def x2_width(self) -> int:
        """Elements of a row of the second operand (and of its gradient) in memory."""
        return 3 if self.harmonics else self.nseg_x2

    @property
    def monomials(self) -> list:
        """The distinct monomials (sorted index tuples, the constant first) of the harmonics."""
        return sorted({vi for terms in self.harmonics for vi, _ in terms}, key=lambda t: (len(t), t))

    @property
    def num_paths(self):
        return sum(len(b.entries) for b in self.blocks)

    def _at(self, layout, seg: int) -> str:
        """Element offset of (segment, this lane's channel ``uu``) inside a row, as a C expression."""
        if not layout:
            return f"{seg * self.extent} + uu"
        off = 0
        for d in layout:
            if seg < d:
                return f"{off + seg} + uu" if d == 1 else f"{off + seg} + uu * {d}"
            seg -= d
            off += d * self.extent
        raise IndexError(seg)

    def x1_at(self, i: int) -> str:
        return self._at(self.layout_x1, i)

    def out_at(self, k: int) -> str:
        return self._at(self.layout_out, k)


def analyze(extent: int, nseg: Sequence[int], paths: Sequence[tuple], layout_x1: tuple = (), layout_out: tuple = (),
            harmonics: tuple = ()) -> ChannelwiseStructure:
    """``paths``: (w_seg, x1_seg, x2_seg, out_seg, coefficient)."""
    blocks: dict[int, Block] = {}
    for b, i, j, k, c in paths:
        if c == 0.0:
            continue
        blocks.setdefault(b, Block(b)).entries.append((i, j, k, float(c)))
    out = [blocks[b] for b in sorted(blocks)]
    # Order blocks so that blocks reading the same x1 segments are neighbours (register reuse).
    out.sort(key=lambda blk: (blk.i_list, blk.j_list, blk.b))
    assert not harmonics or len(harmonics) == nseg[2]
    return ChannelwiseStructure(extent, nseg[0], nseg[1], nseg[2], nseg[3], out, tuple(layout_x1), tuple(layout_out), tuple(harmonics))


def _lit(c: float, T: str) -> str:
    s = repr(float(c))
    if "e" not in s and "." not in s and "inf" not in s and "nan" not in s:
        s += ".0"
    return s + ("f" if T == "float" else "")


def _mono_name(vi: tuple) -> str:
    return "mo_" + "".join(str(i) for i in vi) if vi else "mo_one"


def _emit_monomials(A, ind: str, T: str, monos: Sequence[tuple], v: Sequence[str]):
    """``const T mo_<indices>`` for every monomial of ``monos`` (closed under prefixes, see ``_with_prefixes``), each from its
    prefix by one multiplication."""
    for vi in sorted(monos, key=lambda t: (len(t), t)):
        if not vi:
            A(f"{ind}const {T} mo_one = 1;")
        elif len(vi) == 1:
            A(f"{ind}const {T} {_mono_name(vi)} = {v[vi[0]]};")
        else:
            assert vi[:-1] in monos, (vi, monos)
            A(f"{ind}const {T} {_mono_name(vi)} = {_mono_name(vi[:-1])} * {v[vi[-1]]};")


def _with_prefixes(monos) -> list:
    out = set()
    for vi in monos:
        for n in range(len(vi) + 1):
            out.add(tuple(vi[:n]))
    return sorted(out, key=lambda t: (len(t), t))


# ---------------------------------------------------------------------------------------------
# forward
# ---------------------------------------------------------------------------------------------
def _block_cost(blk: Block) -> int:
    return len(blk.entries) + 2 * len(blk.k_list)


def _split_blocks(st: ChannelwiseStructure, nsplit: int) -> list[list[Block]]:
    """Blocks dealt out to ``nsplit`` groups (one wavefront each) so that no two groups read the same x1 segment: every
    output segment belongs to one block, so groups then share nothing but x2 - each loads its own x1 segments and
    weights, keeps its own accumulators (forward) or cotangent registers (backward) and owns the x1 gradient of its
    segments.  Blocks are first joined into components that share x1 segments (for a channel-wise product: one per
    irrep of the first operand), the components are balanced greedily by path count.  Fewer groups come back when
    there are fewer components."""
    parent = {}

    def find(a):
        while parent.setdefault(a, a) != a:
            parent[a] = parent[parent[a]]
            a = parent[a]
        return a

    for blk in st.blocks:
        first = blk.i_list[0]
        for i in blk.i_list[1:]:
            parent[find(i)] = find(first)
    comps = defaultdict(list)
    for blk in st.blocks:
        comps[find(blk.i_list[0])].append(blk)
    comps = sorted(comps.values(), key=lambda c: -sum(_block_cost(b) for b in c))
    nsplit = max(1, min(nsplit, len(comps)))
    groups = [[] for _ in range(nsplit)]
    load = [0] * nsplit
    for comp in comps:
        g = load.index(min(load))
        groups[g] += comp
        load[g] += sum(_block_cost(b) for b in comp)
    for g in groups:
        g.sort(key=lambda blk: (blk.i_list, blk.j_list, blk.b))
    return groups


def _tables_for(blocks: Sequence[Block]):
    """Assign every path a slot (table t, lane n): n = x2 index mod 16, one Y register per 16 x2 segments.

    Returns (slots: {(b, idx_in_block): (t, n)}, table rows: list of (m, [coeff for n in 0..15])).
    """
    per_j = defaultdict(list)
    for blk in blocks:
        for e_idx, (i, j, k, c) in enumerate(blk.entries):
            per_j[j].append((blk.b, e_idx, c))
    tables = []  # (m, coeffs[16])
    slots = {}
    ms = sorted({j // 16 for j in per_j})
    for m in ms:
        depth = max(len(per_j[j]) for j in per_j if j // 16 == m)
        base = len(tables)
        for t in range(depth):
            tables.append((m, [0.0] * 16))
        for j in per_j:
            if j // 16 != m:
                continue
            for t, (b, e_idx, c) in enumerate(per_j[j]):
                tables[base + t][1][j % 16] = c
                slots[(b, e_idx)] = (base + t, j % 16)
    return slots, tables


def emit_forward(st: ChannelwiseStructure, T: str, nsplit: int, waves_per_eu: int, ns: str, prefetch: bool = True) -> str:
    """HIP source of the forward kernels (one ``__device__`` body per block group) in namespace ``ns``."""
    fp = T
    dpp = "v_fmac_f32_dpp" if T == "float" else "v_fmac_f64_dpp"
    groups = _split_blocks(st, nsplit)
    nsplit = len(groups)
    L = []
    A = L.append
    A(f"// forward: {st.num_paths} paths, {len(st.blocks)} blocks, split over {nsplit} wave group(s)")
    all_tables = []
    group_meta = []
    for q, blocks in enumerate(groups):
        slots, tables = _tables_for(blocks)
        group_meta.append((slots, len(all_tables), len(tables)))
        all_tables += tables
    A(f"__device__ const {fp} fwd_ctab[{max(1, len(all_tables)) * 16}] = {{")
    for m, row in all_tables:
        A("  " + ", ".join(_lit(c, T) for c in row) + ",")
    A("};")
    A(f"constexpr int kFwdTables = {len(all_tables)};")
    monos = st.monomials
    NM = len(monos)
    if st.harmonics:
        # lane n16 evaluates Y_(16 m + n16): its coefficients come from LDS, the monomials of the vector are the same in all lanes
        npad = 16 * ((st.nseg_x2 + 15) // 16)
        A(f"__device__ const {fp} fwd_shtab[{npad * NM}] = {{")
        for j in range(npad):
            row = dict(st.harmonics[j]) if j < st.nseg_x2 else {}
            A("  " + ", ".join(_lit(row.get(vi, 0.0), T) for vi in monos) + ",")
        A("};")
    A("")
    for q, blocks in enumerate(groups):
        slots, tbase, ntab = group_meta[q]
        tables = all_tables[tbase: tbase + ntab]
        ks = sorted({k for blk in blocks for k in blk.k_list})
        i_used = sorted({i for blk in blocks for i in blk.i_list})
        ms = sorted({m for m, _ in tables})

        def load(S: str, zz: str, ind: str):
            A(f"{ind}{{")
            A(f"{ind}  const int64_t z = csr_perm ? csr_perm[{zz}] : ({zz});")
            A(f"{ind}  int64_t srow = z;")
            A(f"{ind}  if (X1_IDX) srow = x1_idx64 ? static_cast<const int64_t*>(x1_index)[z] : static_cast<int64_t>(static_cast<const int32_t*>(x1_index)[z]);")
            A(f"{ind}  const TI* __restrict__ x1p = x1 + srow * {st.nseg_x1 * st.extent}ll;")
            A(f"{ind}  const TI* __restrict__ wp = w + (W_SHARED ? 0 : z * {st.nseg_w * st.extent}ll);")
            A(f"{ind}  const TI* __restrict__ x2p = x2 + z * {st.x2_width}ll;")
            if st.harmonics:
                for a in range(3):
                    A(f"{ind}  {S}_v{a} = io_ld(x2p + {a});")
            for m in ([] if st.harmonics else ms):
                nvalid = min(16, st.nseg_x2 - 16 * m)
                A(f"{ind}  {S}_yv{m} = io_ld(x2p + {16 * m} + (n16 < {nvalid} ? n16 : 0));")
            for i in i_used:
                A(f"{ind}  {S}_xv{i} = io_ld(x1p + ({st.x1_at(i)}));")
            for blk in blocks:
                A(f"{ind}  {S}_wv{blk.b} = io_ldnt(wp + {blk.b * st.extent} + uu);")
            A(f"{ind}}}")

        def body(S: str, ind: str):
            if st.harmonics:
                _emit_monomials(A, ind, fp, _with_prefixes(monos), [f"{S}_v0", f"{S}_v1", f"{S}_v2"])
                for m in ms:
                    expr = None
                    for q_, vi in enumerate(monos):
                        term = f"s_sh[({16 * m} + n16) * {NM} + {q_}]"
                        expr = f"{term} * {_mono_name(vi)}" if expr is None else f"fma({term}, {_mono_name(vi)}, {expr})"
                    A(f"{ind}const {fp} {S}_yv{m} = {expr};")
            for t, (m, _row) in enumerate(tables):
                A(f"{ind}{fp} t{t} = s_c[{(tbase + t) * 16} + n16] * {S}_yv{m};")
            # fence: table registers are produced by VALU and consumed through DPP
            names = [f"t{t}" for t in range(ntab)]
            for c0 in range(0, len(names), 12):
                ops = ", ".join(f'"+v"({n})' for n in names[c0: c0 + 12])
                A(f'{ind}asm volatile("s_nop 1" : {ops});')
            for blk in blocks:
                A(f"{ind}{{  // block w[{blk.b}]: x1 {blk.i_list} x x2 {blk.j_list} -> out {blk.k_list}")
                for i in blk.i_list:
                    A(f"{ind}  const {fp} wx{i} = {S}_wv{blk.b} * {S}_xv{i};")
                for e_idx, (i, j, k, c) in enumerate(blk.entries):
                    t, n = slots[(blk.b, e_idx)]
                    A(f'{ind}  asm("{dpp} %0, %1, %2 row_newbcast:{n} row_mask:0xf bank_mask:0xf" : "+v"(acc{k}) : "v"(t{t}), "v"(wx{i}));')
                A(f"{ind}}}")

        A(f"template <bool X1_IDX, bool W_SHARED>")
        A(f"__device__ __forceinline__ void fwd_group{q}(FWD_PARAMS, const {fp}* s_c, const {fp}* s_sh, int64_t r, int lane, int uu, bool active) {{")
        for k in ks:
            A(f"  {fp} acc{k} = 0;")
        A("  int64_t z0, z1;")
        A("  if (csr_offsets) { z0 = csr_offsets[r]; z1 = csr_offsets[r + 1]; } else { z0 = r; z1 = r + 1; }")
        A("  const int n16 = lane & 15;")
        sets = ("a", "b") if prefetch else ("a",)
        for S in sets:
            second = [f"{S}_v{a} = 0" for a in range(3)] if st.harmonics else [f"{S}_yv{m} = 0" for m in ms]
            A(f"  {fp} " + ", ".join(second + [f"{S}_xv{i} = 0" for i in i_used]
                                      + [f"{S}_wv{blk.b} = 0" for blk in blocks]) + ";")
        if prefetch:
            # The rows of the next batch element are requested before the arithmetic of the current one.  The requests
            # are unconditional (past the end the last element is fetched again): after a conditional request the
            # number of outstanding loads is unknown and the wait before the arithmetic becomes "all of them",
            # the ones just issued included.
            A("  if (z0 < z1) {")
            load("a", "z0", "    ")
            A("    for (int64_t zz = z0; zz < z1; zz += 2) {")
            load("b", "(zz + 1 < z1 ? zz + 1 : z1 - 1)", "      ")
            A("      __builtin_amdgcn_sched_barrier(0);")
            A("      {")
            body("a", "        ")
            A("      }")
            A("      if (zz + 1 >= z1) break;")
            load("a", "(zz + 2 < z1 ? zz + 2 : z1 - 1)", "      ")
            A("      __builtin_amdgcn_sched_barrier(0);")
            A("      {")
            body("b", "        ")
            A("      }")
            A("    }")
            A("  }")
        else:
            A("  for (int64_t zz = z0; zz < z1; ++zz) {")
            load("a", "zz", "    ")
            body("a", "    ")
            A("  }")
        A("  if (active) {")
        A(f"    TI* __restrict__ op = out + r * {st.nseg_out * st.extent}ll;")
        for k in ks:
            A(f"    io_stnt(acc{k}, op + ({st.out_at(k)}));")
        A("  }")
        A("}")
        A("")
    # kernel
    nch = (st.extent + 63) // 64
    A("template <bool X1_IDX, bool W_SHARED>")
    A(f"__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu({waves_per_eu}))) fwd_kernel(FWD_PARAMS) {{")
    A(f"  __shared__ {fp} s_c[{max(1, len(all_tables)) * 16}];")
    A("  const int lane = threadIdx.x;")
    A(f"  for (int i = lane; i < {len(all_tables) * 16}; i += 64) s_c[i] = fwd_ctab[i];")
    if st.harmonics:
        A(f"  __shared__ {fp} s_sh[{npad * NM}];")
        A(f"  for (int i = lane; i < {npad * NM}; i += 64) s_sh[i] = fwd_shtab[i];")
    else:
        A(f"  const {fp}* s_sh = nullptr;")
    A("  __syncthreads();")
    A("  int64_t wid = blockIdx.x;")
    A(f"  const int q = static_cast<int>(wid % {nsplit}); wid /= {nsplit};")
    A(f"  const int ch = static_cast<int>(wid % {nch}); const int64_t r = wid / {nch};")
    if st.extent % 64 == 0:
        A("  const int uu = ch * 64 + lane; constexpr bool active = true;")
    else:
        A(f"  const int u = ch * 64 + lane; const bool active = u < {st.extent}; const int uu = active ? u : 0;")
    A("  switch (q) {")
    for q in range(nsplit):
        A(f"    case {q}: fwd_group{q}<X1_IDX, W_SHARED>(FWD_ARGS, s_c, s_sh, r, lane, uu, active); break;")
    A("  }")
    A("}")
    A(f"constexpr int kFwdSplit = {nsplit};")
    A(f"constexpr int kChunks = {nch};")
    return "\n".join(L)


# ---------------------------------------------------------------------------------------------
# backward
# ---------------------------------------------------------------------------------------------
def emit_backward(st: ChannelwiseStructure, T: str, waves_per_eu: int, chunk: int, prefetch: bool = False, nsplit: int = 1) -> str:
    """HIP source of the fused backward kernel (dw, dx1, dx2 in one pass).

    ``nsplit`` > 1 deals the blocks out to that many wavefronts per (range of batch rows, 64 channels) with disjoint x1
    segments (``_split_blocks``): each holds only the cotangent segments of its own blocks in registers, loads its
    own x1 segments and weights, stores its own weight gradients and owns the x1 gradient of its segments; only the x2
    gradient is shared, as one more partial row per wavefront for the fold that already sums the channel chunks.
    Fewer registers per wavefront, more wavefronts per SIMD.

    With ``prefetch`` the operands of the next batch row (x1 row, weight row, x2 row, indices) are fetched into a second
    register set while the current row is processed."""
    fp = T
    L = []
    A = L.append
    nch = (st.extent + 63) // 64
    groups = _split_blocks(st, nsplit)
    nsplit = len(groups)
    nparts = nch * nsplit
    i_all = sorted({i for blk in st.blocks for i in blk.i_list})
    w_all = sorted({blk.b for blk in st.blocks})
    A(f"// backward: fused dw / dx1 / dx2; every wavefront owns one contiguous, equally sized range of batch rows; the blocks are")
    A(f"// dealt out to {nsplit} wavefront(s) per range and channel chunk")
    for q, blocks in enumerate(groups):
        ks = sorted({k for blk in blocks for k in blk.k_list})
        i_used = sorted({i for blk in blocks for i in blk.i_list})
        j_used = sorted({j for blk in blocks for j in blk.j_list})
        # segments nobody computes (all coefficients zero) are zero-filled by the first wavefront
        i_zero = [i for i in range(st.nseg_x1) if i not in i_all] if q == 0 else []
        w_zero = [b for b in range(st.nseg_w) if b not in w_all] if q == 0 else []

        # channel-major groups of x1 this wavefront owns whole: (first segment, size); their gradient is staged through LDS
        staged, first = [], 0
        for d in st.layout_x1:
            if d > 1 and all(i in i_used for i in range(first, first + d)):
                staged.append((first, d))
            first += d
        staged_segments = {i for i0, d in staged for i in range(i0, i0 + d)}

        def load(S: str, zz: str, ind: str):
            A(f"{ind}{{")
            A(f"{ind}  const int64_t z = {zz};")
            A(f"{ind}  {S}_grow = z;")
            A(f"{ind}  if (G_IDX) {S}_grow = g_idx64 ? static_cast<const int64_t*>(g_index)[z] : static_cast<int64_t>(static_cast<const int32_t*>(g_index)[z]);")
            A(f"{ind}  {S}_srow = z;")
            A(f"{ind}  if (X1_IDX) {S}_srow = x1_idx64 ? static_cast<const int64_t*>(x1_index)[z] : static_cast<int64_t>(static_cast<const int32_t*>(x1_index)[z]);")
            A(f"{ind}  const TI* __restrict__ x1p = x1 + {S}_srow * {st.nseg_x1 * st.extent}ll;")
            A(f"{ind}  const TI* __restrict__ wp = w + z * {st.nseg_w * st.extent}ll;")
            A(f"{ind}  const TI* __restrict__ x2p = x2 + z * {st.x2_width}ll;")
            if st.harmonics:  # (requested first: the harmonics below wait for these three only)
                for a in range(3):
                    A(f"{ind}  {S}_v{a} = io_ld(x2p + {a});")
            for i in i_used:
                A(f"{ind}  {S}_xv{i} = io_ld(x1p + ({st.x1_at(i)}));")
            for blk in blocks:
                A(f"{ind}  {S}_wv{blk.b} = io_ldnt(wp + {blk.b * st.extent} + uu);")
            if st.harmonics:
                A(f"{ind}  {{")
                need = sorted({vi for j in j_used for vi, _ in st.harmonics[j]}, key=lambda t: (len(t), t))
                _emit_monomials(A, ind + "    ", fp, _with_prefixes(need), [f"{S}_v0", f"{S}_v1", f"{S}_v2"])
                for j in j_used:
                    expr = None
                    for vi, c in st.harmonics[j]:
                        expr = f"{_lit(c, T)} * {_mono_name(vi)}" if expr is None else f"fma({_lit(c, T)}, {_mono_name(vi)}, {expr})"
                    A(f"{ind}    {S}_yv{j} = {expr if expr is not None else '0'};")
                A(f"{ind}  }}")
            for j in ([] if st.harmonics else j_used):
                A(f"{ind}  {S}_yv{j} = io_ld(x2p + {j});")
            A(f"{ind}}}")

        def body(S: str, zz: str, ind: str):
            A(f"{ind}const int64_t z = {zz};")
            A(f"{ind}if ({S}_grow != grow_cur) {{")
            A(f"{ind}  grow_cur = {S}_grow;")
            A(f"{ind}  const TI* __restrict__ gp = g + grow_cur * {st.nseg_out * st.extent}ll;")
            for k in ks:
                A(f"{ind}  gr{k} = io_ldnt(gp + ({st.out_at(k)}));")
            A(f"{ind}}}")
            A(f"{ind}TI* __restrict__ dwp = dw + z * {st.nseg_w * st.extent}ll;")
            for i in i_used:
                A(f"{ind}{fp} dxa{i} = 0;")
            for j in j_used:
                A(f"{ind}{fp} pj{j} = 0;")
            for blk in blocks:
                A(f"{ind}{{  // block w[{blk.b}]")
                A(f"{ind}  const {fp} wb = {S}_wv{blk.b};")
                gij = defaultdict(list)
                for i, j, k, c in blk.entries:
                    gij[(i, j)].append((k, c))
                A(f"{ind}  {fp} dwb = 0;")
                for j in blk.j_list:
                    A(f"{ind}  {fp} F{j} = 0;")
                # per x1 component: G = sum_k c g_k is a temporary feeding both D (with x2) and F (with x1)
                for i in blk.i_list:
                    A(f"{ind}  {{")
                    A(f"{ind}    {fp} D = 0;")
                    for j in blk.j_list:
                        if (i, j) not in gij:
                            continue
                        expr = None
                        for k, c in gij[(i, j)]:
                            expr = f"{_lit(c, T)} * gr{k}" if expr is None else f"fma({_lit(c, T)}, gr{k}, {expr})"
                        A(f"{ind}    {{ const {fp} G = {expr}; D = fma(G, {S}_yv{j}, D); F{j} = fma(G, {S}_xv{i}, F{j}); }}")
                    A(f"{ind}    dwb = fma({S}_xv{i}, D, dwb); dxa{i} = fma(wb, D, dxa{i});")
                    A(f"{ind}  }}")
                A(f"{ind}  if (active) io_stnt(dwb, dwp + {blk.b * st.extent} + uu);")
                for j in blk.j_list:
                    A(f"{ind}  pj{j} = fma(wb, F{j}, pj{j});")
                A(f"{ind}}}")
                A(f"{ind}__builtin_amdgcn_sched_barrier(0);")
            for b_ in w_zero:
                A(f"{ind}if (active) io_stnt({fp}(0), dwp + {b_ * st.extent} + uu);")
            # dx1: scatter.  Atomic adds are served per touched 32-byte sector, not per element: the components of a
            # channel-major group (a stride of d elements between lanes) go through LDS first, so that every atomic
            # instruction of the wavefront covers 64 consecutive elements as it does in the default layout.
            for i0, d in staged:
                A(f"{ind}if (ATOMIC_DX1) {{")
                A(f"{ind}  {fp}* dp = dx1 + {S}_srow * {st.nseg_x1 * st.extent}ll + {st.extent * i0} + ch * {64 * d};")
                A(f"{ind}  __builtin_amdgcn_wave_barrier();")
                for c in range(d):
                    A(f"{ind}  dxs[lane * {d} + {c}] = dxa{i0 + c};")
                A(f"{ind}  __builtin_amdgcn_wave_barrier();")
                for k in range(d):
                    guard = "" if st.extent % 64 == 0 else f"if (ch * {64 * d} + {k * 64} + lane < {st.extent * d}) "
                    A(f"{ind}  {guard}unsafeAtomicAdd(dp + {k * 64} + lane, dxs[{k * 64} + lane]);")
                A(f"{ind}}}")
            A(f"{ind}if (active) {{")
            A(f"{ind}  if (ATOMIC_DX1) {{")
            A(f"{ind}    {fp}* dp = dx1 + {S}_srow * {st.nseg_x1 * st.extent}ll;")
            for i in i_used:
                if i not in staged_segments:
                    A(f"{ind}    unsafeAtomicAdd(dp + ({st.x1_at(i)}), dxa{i});")
            A(f"{ind}  }} else {{")
            A(f"{ind}    TI* __restrict__ dp = dx1_partial + z * {st.nseg_x1 * st.extent}ll;")
            for i in sorted(i_used + i_zero):
                A(f"{ind}    io_st(" + (f"dxa{i}" if i in i_used else f"{fp}(0)") + f", dp + ({st.x1_at(i)}));")
            A(f"{ind}  }}")
            A(f"{ind}}}")
            # dx2: reduce over the 64 lanes; channel chunks and wavefronts of one batch row are folded afterwards
            A(f"{ind}if (!active) {{" + " ".join(f"pj{j} = 0;" for j in j_used) + "}")
            for j in j_used:
                A(f"{ind}pj{j} = wave_sum(pj{j});")
            if st.harmonics:
                # dv[a] = sum_j pj[j] dY_j/dv[a] (this wavefront's share: the sum over its channels and blocks is linear)
                rests = set()
                for j in j_used:
                    for vi, _ in st.harmonics[j]:
                        for a in sorted(set(vi)):
                            rest = list(vi)
                            rest.remove(a)
                            rests.add(tuple(rest))
                A(f"{ind}{fp} dv0 = 0, dv1 = 0, dv2 = 0;")
                A(f"{ind}{{")
                _emit_monomials(A, ind + "  ", fp, _with_prefixes(rests), [f"{S}_v0", f"{S}_v1", f"{S}_v2"])
                for j in j_used:
                    for vi, c in st.harmonics[j]:
                        for a in sorted(set(vi)):
                            rest = list(vi)
                            rest.remove(a)
                            A(f"{ind}  dv{a} = fma({_lit(c * vi.count(a), T)} * pj{j}, {_mono_name(tuple(rest))}, dv{a});")
                A(f"{ind}}}")
            A(f"{ind}if (lane == 0) {{")
            if nparts == 1:
                A(f"{ind}  TI* __restrict__ d2 = dx2 + z * {st.x2_width}ll;")
            else:
                A(f"{ind}  {fp}* __restrict__ d2 = dx2_partial + (z * {nparts} + ch * {nsplit} + {q}) * {st.x2_width}ll;")
            if st.harmonics:
                for a in range(3):
                    A(f"{ind}  io_st(dv{a}, d2 + {a});")
            else:
                for j in range(st.nseg_x2):
                    A(f"{ind}  io_st(" + (f"pj{j}" if j in j_used else f"{fp}(0)") + f", d2 + {j});")
            A(f"{ind}}}")

        A("template <bool X1_IDX, bool G_IDX, bool ATOMIC_DX1>")
        A(f"__device__ __forceinline__ void bwd_group{q}(BWD_PARAMS, int64_t z0, int64_t z1, int lane, int uu, bool active, int ch) {{")
        if staged:
            A(f"  __shared__ {fp} dxs[{64 * max(d for _, d in staged)}];")
        for k in ks:
            A(f"  {fp} gr{k} = 0;")
        A("  int64_t grow_cur = -1;")
        sets = ("a", "b") if prefetch else ("a",)
        for S in sets:
            A(f"  int64_t {S}_grow = -1, {S}_srow = 0;")
            A(f"  {fp} " + ", ".join([f"{S}_xv{i} = 0" for i in i_used] + [f"{S}_wv{blk.b} = 0" for blk in blocks]
                                      + [f"{S}_yv{j} = 0" for j in j_used]
                                      + ([f"{S}_v{a} = 0" for a in range(3)] if st.harmonics else [])) + ";")
        if prefetch:
            # one copy of the body (two copies drive the register allocator into hundreds of spills): set "a" is the row in
            # work, set "b" the row being fetched; "a = b" at the end of the iteration
            A("  if (z0 < z1) {")
            load("a", "z0", "    ")
            A("  }")
            A("  for (int64_t zz = z0; zz < z1; ++zz) {")
            A("    {")
            load("b", "(zz + 1 < z1 ? zz + 1 : zz)", "      ")
            A("    }")
            A("    __builtin_amdgcn_sched_barrier(0);")
            A("    {")
            body("a", "zz", "      ")
            A("    }")
            A("    a_grow = b_grow; a_srow = b_srow;")
            A("    " + " ".join([f"a_xv{i} = b_xv{i};" for i in i_used] + [f"a_wv{blk.b} = b_wv{blk.b};" for blk in blocks]
                                 + [f"a_yv{j} = b_yv{j};" for j in j_used]
                                 + ([f"a_v{a} = b_v{a};" for a in range(3)] if st.harmonics else [])))
            A("  }")
        else:
            A("  for (int64_t zz = z0; zz < z1; ++zz) {")
            load("a", "zz", "    ")
            A("    {")
            body("a", "zz", "      ")
            A("    }")
            A("  }")
        A("}")
        A("")
    A("template <bool X1_IDX, bool G_IDX, bool ATOMIC_DX1>")
    A(f"__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu({waves_per_eu}))) bwd_kernel(BWD_PARAMS) {{")
    A("  const int lane = threadIdx.x;")
    A("  int64_t wid = blockIdx.x;")
    A(f"  const int q = static_cast<int>(wid % {nsplit}); wid /= {nsplit};")
    A(f"  const int ch = static_cast<int>(wid % {nch}); const int64_t cid = wid / {nch};")
    if st.extent % 64 == 0:
        A("  const int uu = ch * 64 + lane; constexpr bool active = true;")
    else:
        A(f"  const int u = ch * 64 + lane; const bool active = u < {st.extent}; const int uu = active ? u : 0;")
    A(f"  const int64_t nranges = gridDim.x / {nparts};")
    A("  const int64_t z0 = cid * batch / nranges, z1 = (cid + 1) * batch / nranges;")
    A("  switch (q) {")
    for q in range(nsplit):
        A(f"    case {q}: bwd_group{q}<X1_IDX, G_IDX, ATOMIC_DX1>(BWD_ARGS, z0, z1, lane, uu, active, ch); break;")
    A("  }")
    A("}")
    A(f"constexpr int kBwdMinRange = {chunk};   // fewest batch rows worth a wavefront of their own")
    A(f"constexpr int kBwdWaves = {waves_per_eu};")
    A(f"constexpr int kBwdSplit = {nsplit};")
    A(f"constexpr int kBwdParts = {nparts};     // partial rows of the x2 gradient per batch row")
    return "\n".join(L)



# ---------------------------------------------------------------------------------------------
# translation unit
# ---------------------------------------------------------------------------------------------
FWD_PARAMS = ("const TI* __restrict__ w, const TI* __restrict__ x1, const TI* __restrict__ x2, TI* __restrict__ out, "
              "const void* __restrict__ x1_index, int x1_idx64, const int64_t* __restrict__ csr_offsets, "
              "const int64_t* __restrict__ csr_perm")
FWD_ARGS = "w, x1, x2, out, x1_index, x1_idx64, csr_offsets, csr_perm"
BWD_ARGS = "w, x1, x2, g, dw, dx1, dx1_partial, dx2, dx2_partial, x1_index, x1_idx64, g_index, g_idx64, batch"
# (dx1: sums by atomic additions, dx2_partial: partial rows - both in the arithmetic type; everything else holds TI)
BWD_PARAMS = ("const TI* __restrict__ w, const TI* __restrict__ x1, const TI* __restrict__ x2, const TI* __restrict__ g, "
              "TI* __restrict__ dw, {T}* dx1, TI* __restrict__ dx1_partial, TI* __restrict__ dx2, "
              "{T}* __restrict__ dx2_partial, const void* __restrict__ x1_index, int x1_idx64, "
              "const void* __restrict__ g_index, int g_idx64, int64_t batch")


IO_TYPES = {"bf16": ("bf16_t", "CUEQ_BF16"), "f16": ("f16_t", "CUEQ_F16")}


def io_type(T: str, io) -> tuple:
    """(C++ element type of the buffers, its CUEQ_* code, tag for names) of a unit computing in ``T`` whose buffers hold
    ``io`` (None: ``T`` itself; "bf16" / "f16": 16-bit elements, float arithmetic only)."""
    if io is None:
        return T, ("CUEQ_F32" if T == "float" else "CUEQ_F64"), T
    if T != "float" or io not in IO_TYPES:
        raise ValueError(f"buffers of {io} with {T} arithmetic are not generated")
    return (*IO_TYPES[io], io)


def emit_unit(st: ChannelwiseStructure, T: str, name: str, fwd_hash: int, bwd_hash: int, *, fwd_split: int = 1,
              fwd_waves: int = 2, fwd_prefetch: bool = True, bwd_waves: int = 2, bwd_chunk: int = 16,
              bwd_prefetch: bool = False, bwd_split: int = 1, io=None) -> str:
    """Complete .hip translation unit: kernels, host launchers, registration under both table hashes.  ``io``: element type
    of the buffers when it is not the arithmetic type ``T`` ("bf16" / "f16" with ``T`` = float)."""
    TI, io_code, tag = io_type(T, io)
    ns = f"cw_{name}" + (f"_{tag}" if io else "")
    nch = (st.extent + 63) // 64
    W1, WW, W2, WO = st.nseg_x1 * st.extent, st.nseg_w * st.extent, st.x2_width, st.nseg_out * st.extent
    out = []
    A = out.append
    A("// GENERATED by cuequivariance_amd/codegen/channelwise.py - do not edit.")
    A(f"// channel-wise tensor product '{name}': extent {st.extent}, segments w/x1/x2/out = "
      f"{st.nseg_w}/{st.nseg_x1}/{st.nseg_x2}/{st.nseg_out}, {st.num_paths} paths, math {T}"
      + (f", buffers of {tag}" if io else "")
      + (f", x1 rows in groups {list(st.layout_x1)}" if st.layout_x1 else "") + (f", output rows in groups {list(st.layout_out)}" if st.layout_out else "")
      + (", x2 = spherical harmonics of a 3-vector evaluated in the kernels" if st.harmonics else ""))
    A('#include "cw_common.h"')
    A("")
    A("namespace cueq {")
    A(f"namespace {ns} {{")
    A(f"using TI = {TI};  // element type of the buffers; operands read or written exactly once per launch (weights, weight")
    A("// gradients, output rows) go through io_ldnt / io_stnt so that they do not displace the gathered rows in the caches")
    A(f"#define FWD_PARAMS {FWD_PARAMS.format(T=T)}")
    A(f"#define FWD_ARGS {FWD_ARGS}")
    A(f"#define BWD_PARAMS {BWD_PARAMS.format(T=T)}")
    A(f"#define BWD_ARGS {BWD_ARGS}")
    A("")
    A(emit_forward(st, T, fwd_split, fwd_waves, ns, fwd_prefetch))
    A("")
    A(emit_backward(st, T, bwd_waves, bwd_chunk, bwd_prefetch, bwd_split))
    A("")
    same = "true" if io is None else "false"
    A(f"""
constexpr bool kSameType = {same};  // buffers hold the arithmetic type

// buffers: w, x1, x2 | out
static int run_fwd(const SpecCall& c) {{
  const cueq_u1d_buffer* b = c.buffers;
  if (common_dtype(b, 4) != {io_code}) return CUEQ_ERR_UNSUPPORTED;
  if (b[2].batch_dim != CUEQ_BATCH_BATCHED) return CUEQ_ERR_UNSUPPORTED;
  if (b[0].batch_dim == CUEQ_BATCH_INDEXED || b[1].batch_dim == CUEQ_BATCH_SHARED) return CUEQ_ERR_UNSUPPORTED;
  if (b[3].batch_dim == CUEQ_BATCH_SHARED) return CUEQ_ERR_UNSUPPORTED;
  const bool x1_idx = b[1].batch_dim == CUEQ_BATCH_INDEXED, w_shared = b[0].batch_dim == CUEQ_BATCH_SHARED;
  const bool out_idx = b[3].batch_dim == CUEQ_BATCH_INDEXED;
  if (out_idx && (!b[3].csr_offsets || (!b[3].csr_perm && c.batch > 0))) return CUEQ_ERR_UNSUPPORTED;
  const int64_t rows = b[3].rows;
  if (rows == 0) return CUEQ_OK;
  const int64_t grid = rows * {nch} * kFwdSplit;
  CUEQ_REQUIRE(grid < (int64_t(1) << 31), CUEQ_ERR_TOO_LARGE, "too many output rows for one launch");
  const TI* w = static_cast<const TI*>(b[0].data);
  const TI* x1 = static_cast<const TI*>(b[1].data);
  const TI* x2 = static_cast<const TI*>(b[2].data);
  TI* o = static_cast<TI*>(b[3].data);
  const int64_t* offs = out_idx ? b[3].csr_offsets : nullptr;
  const int64_t* perm = out_idx ? b[3].csr_perm : nullptr;
  const dim3 g(static_cast<unsigned>(grid)), t(64);
  KernelTimer timer("{name}_fwd_{tag}", c.stream);
#define LAUNCH_FWD(XI, WS) hipLaunchKernelGGL((fwd_kernel<XI, WS>), g, t, 0, c.stream, w, x1, x2, o, b[1].index, b[1].index_is_64, offs, perm)
  if (x1_idx && w_shared) LAUNCH_FWD(true, true);
  else if (x1_idx) LAUNCH_FWD(true, false);
  else if (w_shared) LAUNCH_FWD(false, true);
  else LAUNCH_FWD(false, false);
#undef LAUNCH_FWD
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}}

// buffers: w, x1, x2, g | dw, dx1, dx2
// workspace: [partial rows of the x2 gradient, arithmetic type] [the x1 gradient of a gathered operand: one partial row per
// batch row in TI (summed in index order afterwards), or - for 16-bit buffers and atomic sums - its rows in the arithmetic type]
static int64_t bwd_workspace(const cueq_u1d_buffer* b, int64_t batch) {{
  if (common_dtype(b, 7) != {io_code}) return 0;
  int64_t need = 0;
  if (kBwdParts > 1) need += batch * kBwdParts * {W2}ll * sizeof({T});
  need = (need + 255) & ~int64_t(255);
  if (b[1].batch_dim == CUEQ_BATCH_INDEXED) {{
    if (deterministic_scatter()) need += batch * {W1}ll * sizeof(TI);
    else if (!kSameType) need += b[5].rows * {W1}ll * sizeof({T});
  }}
  return need;
}}

static int run_bwd(const SpecCall& c) {{
  const cueq_u1d_buffer* b = c.buffers;
  if (common_dtype(b, 7) != {io_code}) return CUEQ_ERR_UNSUPPORTED;
  if (b[0].batch_dim != CUEQ_BATCH_BATCHED || b[2].batch_dim != CUEQ_BATCH_BATCHED) return CUEQ_ERR_UNSUPPORTED;
  if (b[1].batch_dim == CUEQ_BATCH_SHARED || b[3].batch_dim == CUEQ_BATCH_SHARED) return CUEQ_ERR_UNSUPPORTED;
  if (b[4].batch_dim != CUEQ_BATCH_BATCHED || b[6].batch_dim != CUEQ_BATCH_BATCHED) return CUEQ_ERR_UNSUPPORTED;
  if (b[5].batch_dim != b[1].batch_dim) return CUEQ_ERR_UNSUPPORTED;
  const bool x1_idx = b[1].batch_dim == CUEQ_BATCH_INDEXED, g_idx = b[3].batch_dim == CUEQ_BATCH_INDEXED;
  if (x1_idx && (b[5].index != b[1].index || b[5].rows != b[1].rows)) return CUEQ_ERR_UNSUPPORTED;
  const bool det = deterministic_scatter();
  if (x1_idx && det && (!b[5].csr_offsets || (!b[5].csr_perm && c.batch > 0))) return CUEQ_ERR_UNSUPPORTED;
  const int64_t batch = c.batch;
  const TI* w = static_cast<const TI*>(b[0].data);
  const TI* x1 = static_cast<const TI*>(b[1].data);
  const TI* x2 = static_cast<const TI*>(b[2].data);
  const TI* g = static_cast<const TI*>(b[3].data);
  TI* dw = static_cast<TI*>(b[4].data);
  TI* dx1 = static_cast<TI*>(b[5].data);
  TI* dx2 = static_cast<TI*>(b[6].data);
  const int64_t need = bwd_workspace(b, batch);
  CUEQ_REQUIRE(need == 0 || (c.workspace && c.workspace_bytes >= need), CUEQ_ERR_INVALID, "workspace too small: need %lld bytes", (long long)need);
  char* ws = static_cast<char*>(c.workspace);
  {T}* dx2_partial = nullptr;
  int64_t off = 0;
  if (kBwdParts > 1) {{ dx2_partial = reinterpret_cast<{T}*>(ws); off = (batch * kBwdParts * {W2}ll * sizeof({T}) + 255) & ~int64_t(255); }}
  TI* dx1_partial = nullptr;
  {T}* dx1_sums = nullptr;  // target of the atomic additions
  if (!x1_idx) dx1_partial = dx1;  // one row per batch element: plain stores
  else if (det) dx1_partial = reinterpret_cast<TI*>(ws + off);
  else dx1_sums = kSameType ? reinterpret_cast<{T}*>(dx1) : reinterpret_cast<{T}*>(ws + off);
  const bool atomic = dx1_sums != nullptr;
  if (atomic && b[5].rows > 0) {{
    const int64_t n = b[5].rows * {W1}ll;
    hipLaunchKernelGGL(fill_zero<{T}>, dim3(fill_blocks<{T}>(n)), dim3(256), 0, c.stream, dx1_sums, n);
    CUEQ_CHECK_HIP(hipGetLastError());
  }}
  if (batch > 0) {{
    // one launch round of resident wavefronts; short batches get fewer, not shorter than kBwdMinRange rows
    int64_t nranges = wave_slots(kBwdWaves) / kBwdParts;
    const int64_t most = (batch + kBwdMinRange - 1) / kBwdMinRange;
    if (nranges > most) nranges = most;
    if (nranges < 1) nranges = 1;
    const int64_t grid = nranges * kBwdParts;
    const dim3 gd(static_cast<unsigned>(grid)), t(64);
    {{
    KernelTimer timer("{name}_bwd_{tag}", c.stream);
#define LAUNCH_BWD(XI, GI, AT) hipLaunchKernelGGL((bwd_kernel<XI, GI, AT>), gd, t, 0, c.stream, w, x1, x2, g, dw, dx1_sums, dx1_partial, dx2, dx2_partial, b[1].index, b[1].index_is_64, b[3].index, b[3].index_is_64, batch)
    if (x1_idx && g_idx && atomic) LAUNCH_BWD(true, true, true);
    else if (x1_idx && g_idx) LAUNCH_BWD(true, true, false);
    else if (x1_idx && atomic) LAUNCH_BWD(true, false, true);
    else if (x1_idx) LAUNCH_BWD(true, false, false);
    else if (g_idx) LAUNCH_BWD(false, true, false);
    else LAUNCH_BWD(false, false, false);
#undef LAUNCH_BWD
    }}
    CUEQ_CHECK_HIP(hipGetLastError());
    if (kBwdParts > 1) {{
      hipLaunchKernelGGL((fold_parts<{T}, TI>), dim3(blocks_for(batch * {W2}ll)), dim3(256), 0, c.stream, dx2_partial, batch, kBwdParts, {W2}, dx2);
      CUEQ_CHECK_HIP(hipGetLastError());
    }}
  }}
  if (atomic && !kSameType && b[5].rows > 0) {{
    const int64_t n = b[5].rows * {W1}ll;
    hipLaunchKernelGGL((round_rows<{T}, TI>), dim3(blocks_for(n)), dim3(256), 0, c.stream, dx1_sums, n, dx1);
    CUEQ_CHECK_HIP(hipGetLastError());
  }}
  if (x1_idx && det && b[5].rows > 0) {{
    const int64_t n = b[5].rows * {W1}ll;
    if ({W1} % 4 == 0 && reinterpret_cast<uintptr_t>(dx1) % (4 * sizeof(TI)) == 0 && reinterpret_cast<uintptr_t>(dx1_partial) % (4 * sizeof(TI)) == 0 &&
        b[5].rows < 65536) {{
      hipLaunchKernelGGL(segment_sum_rows_vec<TI>, dim3(({W1} / 4 + 255) / 256, static_cast<unsigned>(b[5].rows)), dim3(256), 0, c.stream,
                         dx1_partial, b[5].csr_offsets, b[5].csr_perm, {W1}, dx1);
    }} else {{
      hipLaunchKernelGGL(segment_sum_rows<TI>, dim3(blocks_for(n)), dim3(256), 0, c.stream, dx1_partial, b[5].csr_offsets, b[5].csr_perm, b[5].rows, {W1}, dx1);
    }}
    CUEQ_CHECK_HIP(hipGetLastError());
  }}
  return CUEQ_OK;
}}

static const U1dSpec spec_fwd = {{0x{fwd_hash:016x}ull, "{name}_fwd_{tag}", run_fwd, nullptr, {io_code}}};
static const U1dSpec spec_bwd = {{0x{bwd_hash:016x}ull, "{name}_bwd_{tag}", run_bwd, bwd_workspace, {io_code}}};
static SpecRegistrar reg_fwd(&spec_fwd);
static SpecRegistrar reg_bwd(&spec_bwd);
""")
    A(f"}}  // namespace {ns}")
    A("}  // namespace cueq")
    return "\n".join(out) + "\n"
