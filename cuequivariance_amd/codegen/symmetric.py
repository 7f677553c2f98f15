"""Generator of straight-line HIP kernels for one symmetric contraction descriptor.

Input: the flattened polynomial ``w[u], x[u] -> out[u]`` with operations ``(w, x, out)``, ``(w, x, x, out)``, ... of
``cuequivariance_amd.cue.descriptors.symmetric_contraction``.  Because the same ``x`` enters every slot, the paths
are first folded onto sorted index tuples (``unsymmetrize_for_identical_operands``: 1949 -> 425 terms of degree 3
for ``128x(0e+1o+2e+3o) -> 128x(0e+1o)``), then grouped by ``(weight segment, output segment)``::

    out[k] = sum_groups w[s] * P_{s,k}(x),     P_{s,k}(x) = sum_terms c * x[a] x[b] x[c]

Forward kernel: one wavefront per resident slot walks a contiguous range of batch rows for 64 channels (lane =
channel); per row it loads the ``x`` segments and the weight row chosen by the row's index, forms the pair products
once, evaluates every group polynomial with literal coefficients and stores the output segments.

Backward kernel (gradients of ``w`` and ``x`` in one pass): walks the rows in the order of the CSR grouping by weight
index, so that consecutive rows share the weight row.  Per term with ``s = c * w[s] * g[k]``:
``dx[a] += s x[b] x[c]`` (and the two rotations), and ``Q[s] += g[k] * P_{s,k}(x)`` accumulates the weight gradient
in registers across rows of the same index.  A wavefront writes ``Q`` directly when a whole index group lies inside
its range and otherwise leaves a head / tail partial that a small fold kernel sums in slot order: no atomics,
bit-reproducible.
"""

from __future__ import annotations

from collections import defaultdict
from dataclasses import dataclass

from .channelwise import _lit, io_type


@dataclass
class SymmetricStructure:
    extent: int
    nseg_w: int
    nseg_x: int
    nseg_out: int
    terms: list  # (weight segment, tuple of sorted x segments, output segment, coefficient)
    layout_x: tuple = ()    # groups of x segments stored channel-major (``U1dTables.layouts``), () = segment-major rows
    layout_out: tuple = ()  # the same for the output rows

    def _at(self, layout: tuple, seg: int) -> str:
        """Element (segment ``seg``, channel ``uu``) of a row under ``layout``, as a C expression."""
        if not layout:
            return f"{seg * self.extent} + uu"
        first = 0
        for d in layout:
            if seg < first + d:
                return f"{first * self.extent + (seg - first)} + uu" + (f" * {d}" if d > 1 else "")
            first += d
        raise ValueError(f"segment {seg} outside the layout {layout}")

    def x_at(self, a: int) -> str:
        return self._at(self.layout_x, a)

    @staticmethod
    def _staged(layout: tuple) -> dict:
        """{segment: (first segment of its group, group size, position in the group)} for groups of more than one segment."""
        out, first = {}, 0
        for d in layout:
            if d > 1:
                for c in range(d):
                    out[first + c] = (first, d, c)
            first += d
        return out

    def out_at(self, k: int) -> str:
        return self._at(self.layout_out, k)

    @property
    def degree(self) -> int:
        return max(len(t[1]) for t in self.terms)


def analyze(poly, layout_x: tuple = (), layout_out: tuple = ()) -> SymmetricStructure:
    """``poly``: the SegmentedPolynomial of a symmetric contraction (modes flattened, ``u`` uniform); the layouts are those
    of the x and output buffers of its tables."""
    assert poly.num_inputs == 2 and poly.num_outputs == 1
    folded = poly.unsymmetrize_for_identical_operands()
    w, x = folded.inputs
    (out,) = folded.outputs
    extent = x.segments[0][0]
    assert all(s == (extent,) for ope in (w, x, out) for s in ope.segments)
    terms = []
    for ope, stp in folded.operations:
        bufs = tuple(ope.buffers)
        assert bufs[0] == 0 and bufs[-1] == 2 and all(b == 1 for b in bufs[1:-1]), bufs
        for path in stp.paths:
            c = float(path.coefficients)
            if c != 0.0:
                terms.append((path.indices[0], tuple(sorted(path.indices[1:-1])), path.indices[-1], c))
    return SymmetricStructure(extent, w.num_segments, x.num_segments, out.num_segments, terms, tuple(layout_x), tuple(layout_out))


def _groups(st: SymmetricStructure):
    g = defaultdict(list)
    for s, xs, k, c in st.terms:
        g[(s, k)].append((xs, c))
    return sorted(g.items())


def _pairs(st: SymmetricStructure):
    pairs = set()
    for _, xs, _, _ in st.terms:
        if len(xs) == 2:
            pairs.add(xs)
        elif len(xs) == 3:
            pairs.update({(xs[0], xs[1]), (xs[0], xs[2]), (xs[1], xs[2])})
        elif len(xs) > 3:
            raise NotImplementedError("generated symmetric contraction kernels cover degrees 1 to 3")
    return sorted(pairs)


def _poly_expr(terms, T: str) -> list[str]:
    """Statements evaluating ``P = sum c * monomial`` with degree-3 terms factored by their last index."""
    lines = [f"{T} P = 0;"]
    by_last = defaultdict(list)
    for xs, c in terms:
        if len(xs) == 1:
            lines.append(f"P = fma({_lit(c, T)}, xv{xs[0]}, P);")
        elif len(xs) == 2:
            lines.append(f"P = fma({_lit(c, T)}, pp_{xs[0]}_{xs[1]}, P);")
        else:
            by_last[xs[2]].append((xs[0], xs[1], c))
    for last, lst in sorted(by_last.items()):
        expr = None
        for a, b, c in lst:
            expr = f"{_lit(c, T)} * pp_{a}_{b}" if expr is None else f"fma({_lit(c, T)}, pp_{a}_{b}, {expr})"
        lines.append(f"P = fma(xv{last}, {expr}, P);")
    return lines


# A channel-major group of d segments is a contiguous piece of 64 d elements per wavefront.  Lanes that each walk their own
# d elements make every load or store instruction touch d times the cache lines it uses, which the address units pay for in
# full; so the piece moves as d unit-stride instructions and crosses the lanes through LDS (lane * d + c <-> k * 64 + lane:
# conflict-free for odd d).  `stage` is private to the wavefront, whose LDS operations execute in program order.
def _piece(st: SymmetricStructure, first: int, d: int, k: int) -> str:
    return f"{first * st.extent} + ch * {64 * d} + {k * 64} + lane"


def _piece_ok(st: SymmetricStructure, d: int, k: int) -> str:
    return "" if st.extent % 64 == 0 else f"(ch * {64 * d} + {k * 64} + lane < {st.extent * d})"


def _row_request(A, ind: str, st: SymmetricStructure, T: str, layout: tuple, segs, ptr: str, dst: str, declare: bool):
    """Loads of the segments `segs` of a row into `dst<seg>`: the value itself for unit-stride segments, for a segment of a
    channel-major group the k-th unit-stride piece of its group (to be unpacked by `_row_unpack`)."""
    staged = st._staged(layout)
    decl = f"const {T} " if declare else ""
    for a in segs:
        if a in staged:
            first, d, k = staged[a]
            ok = _piece_ok(st, d, k)
            load = f"io_ldnt({ptr} + {_piece(st, first, d, k)})"
            A(f"{ind}{decl}{dst}{a} = " + (f"{ok} ? {load} : {T}(0);" if ok else f"{load};"))
        else:
            A(f"{ind}{decl}{dst}{a} = io_ldnt({ptr} + {a * st.extent} + uu);")


def _row_unpack(A, ind: str, st: SymmetricStructure, T: str, layout: tuple, segs, src: str, dst: str):
    """`dst<seg>` = the value of segment `seg` for this lane's channel, from what `_row_request` loaded into `src<seg>`."""
    staged = st._staged(layout)
    done = set()
    for a in segs:
        if a not in staged:
            A(f"{ind}const {T} {dst}{a} = {src}{a};")
            continue
        first, d, _ = staged[a]
        if first in done:
            continue
        done.add(first)
        for k in range(d):
            A(f"{ind}stage[{k * 64} + lane] = {src}{first + k};")
        A(f"{ind}__builtin_amdgcn_wave_barrier();")
        for c in range(d):
            A(f"{ind}const {T} {dst}{first + c} = stage[lane * {d} + {c}];")
        A(f"{ind}__builtin_amdgcn_wave_barrier();")


def _row_store(A, ind: str, st: SymmetricStructure, T: str, layout: tuple, nseg: int, ptr: str, value):
    """Stores of a whole row; `value(seg)` is the expression of this lane's element of segment `seg`."""
    staged = st._staged(layout)
    done = set()
    for a in range(nseg):
        if a not in staged:
            A(f"{ind}if (active) io_stnt({value(a)}, {ptr} + {a * st.extent} + uu);")
            continue
        first, d, _ = staged[a]
        if first in done:
            continue
        done.add(first)
        for c in range(d):
            A(f"{ind}stage[lane * {d} + {c}] = {value(first + c)};")
        A(f"{ind}__builtin_amdgcn_wave_barrier();")
        for k in range(d):
            ok = _piece_ok(st, d, k)
            A(f"{ind}" + (f"if {ok} " if ok else "") + f"io_stnt(stage[{k * 64} + lane], {ptr} + {_piece(st, first, d, k)});")
        A(f"{ind}__builtin_amdgcn_wave_barrier();")


def _whole_groups(layout: tuple, segs, nseg: int):
    """`segs` widened so that every channel-major group it meets is complete."""
    staged = SymmetricStructure._staged(layout)
    out = set(segs)
    for a in segs:
        if a in staged:
            first, d, _ = staged[a]
            out.update(range(first, first + d))
    return sorted(out)


def emit_unit(st: SymmetricStructure, T: str, name: str, fwd_hash: int, bwd_hashes: dict, *, fwd_waves: int = 4,
              bwd_waves: int = 2, fwd_prefetch: bool = None, io=None) -> str:
    """Complete translation unit.  ``bwd_hashes``: {(need_dw, need_dx): table hash}.  ``io``: element type of the buffers when
    it is not the arithmetic type ``T`` ("bf16" / "f16" with ``T`` = float)."""
    TI, io_code, tag = io_type(T, io)
    if fwd_prefetch is None:
        # float: 96 -> 119 registers, still 4 wavefronts per SIMD; double: the pair products alone exceed the register file
        # (the kernel spills either way), a second set of x rows only adds to that
        fwd_prefetch = T == "float"
    ns = f"sc_{name}" + (f"_{tag}" if io else "")
    E, W, X, O = st.extent, st.nseg_w * st.extent, st.nseg_x * st.extent, st.nseg_out * st.extent
    nch = (E + 63) // 64
    groups = _groups(st)
    pairs = _pairs(st)
    x_used = sorted({a for _, xs, _, _ in st.terms for a in xs})
    x_read = _whole_groups(st.layout_x, x_used, st.nseg_x)   # (a group is loaded whole, as its unit-stride pieces)
    w_used = sorted({s for s, _, _, _ in st.terms})
    dmax = max([d for d in tuple(st.layout_x) + tuple(st.layout_out) if d > 1], default=0)
    stage_decl = f"  __shared__ {T} stage[{64 * dmax}];" if dmax else None
    L = []
    A = L.append
    A("// GENERATED by cuequivariance_amd/codegen/symmetric.py - do not edit.")
    A(f"// symmetric contraction '{name}': extent {E}, segments w/x/out = {st.nseg_w}/{st.nseg_x}/{st.nseg_out}, "
      f"{len(st.terms)} folded terms in {len(groups)} (weight, output) groups, math {T}" + (f", buffers of {tag}" if io else "")
      + (f", x rows in groups {list(st.layout_x)}" if st.layout_x else "") + (f", output rows in groups {list(st.layout_out)}" if st.layout_out else ""))
    A('#include "cw_common.h"')
    A("")
    A("namespace cueq {")
    A(f"namespace {ns} {{")
    A(f"using TI = {TI};  // element type of the buffers")
    A("")
    if E % 64 == 0:
        lane_setup = "  const int uu = ch * 64 + lane; constexpr bool active = true;"
    else:
        lane_setup = f"  const int u = ch * 64 + lane; const bool active = u < {E}; const int uu = active ? u : 0;"

    # ------------------------------------------------------------------ forward
    A("// W_MODE: 0 one weight row per batch row, 1 weight row chosen by w_index, 2 a single shared weight row")
    A("template <int W_MODE>")
    A(f"__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu({fwd_waves}))) fwd_kernel(")
    A(f"    const TI* __restrict__ w, const TI* __restrict__ x, TI* __restrict__ out, const void* __restrict__ w_index, int idx64, int64_t batch) {{")
    A("  const int lane = threadIdx.x;")
    A(f"  const int ch = blockIdx.x % {nch}; const int64_t slot = blockIdx.x / {nch}; const int64_t nslots = gridDim.x / {nch};")
    A(lane_setup)
    if stage_decl:
        A(stage_decl)
    A("  const int64_t z0 = slot * batch / nslots, z1 = (slot + 1) * batch / nslots;")
    if fwd_prefetch:
        # the x row (and the weight index) of the next batch row are requested before the arithmetic of the current one; the
        # request is unconditional (the last row is fetched again) so that the waits can count outstanding loads
        A("  if (z0 >= z1) return;")
        A("  int64_t wrow_n = W_MODE == 0 ? z0 : 0;")
        A("  if (W_MODE == 1) wrow_n = load_index(w_index, idx64, z0);")
        A(f"  {T} " + ", ".join(f"xn{a}" for a in x_read) + ";")
        A("  {")
        A(f"    const TI* __restrict__ xp = x + z0 * {X}ll;")
        _row_request(A, "    ", st, T, st.layout_x, x_read, "xp", "xn", False)
        A("  }")
        A("  for (int64_t z = z0; z < z1; ++z) {")
        A("    const int64_t wrow = wrow_n;")
        A(f"    const TI* __restrict__ wp = w + wrow * {W}ll;")
        for s in w_used:
            A(f"    const {T} wv{s} = io_ld(wp + {s * E} + uu);")
        _row_unpack(A, "    ", st, T, st.layout_x, x_read, "xn", "xv")
        A("    {")
        A("      const int64_t zn = z + 1 < z1 ? z + 1 : z;")
        A("      wrow_n = W_MODE == 0 ? zn : 0;")
        A("      if (W_MODE == 1) wrow_n = load_index(w_index, idx64, zn);")
        A(f"      const TI* __restrict__ xp = x + zn * {X}ll;")
        _row_request(A, "      ", st, T, st.layout_x, x_read, "xp", "xn", False)
        A("    }")
        A("    __builtin_amdgcn_sched_barrier(0);")
    else:
        A("  for (int64_t z = z0; z < z1; ++z) {")
        A("    int64_t wrow = W_MODE == 0 ? z : 0;")
        A("    if (W_MODE == 1) wrow = load_index(w_index, idx64, z);")
        A(f"    const TI* __restrict__ xp = x + z * {X}ll;")
        A(f"    const TI* __restrict__ wp = w + wrow * {W}ll;")
        _row_request(A, "    ", st, T, st.layout_x, x_read, "xp", "xr", True)
        for s in w_used:
            A(f"    const {T} wv{s} = io_ld(wp + {s * E} + uu);")
        _row_unpack(A, "    ", st, T, st.layout_x, x_read, "xr", "xv")
    for a, b in pairs:
        A(f"    const {T} pp_{a}_{b} = xv{a} * xv{b};")
    for k in range(st.nseg_out):
        A(f"    {T} acc{k} = 0;")
    for (s, k), terms in groups:
        A(f"    {{  // w[{s}] -> out[{k}], {len(terms)} terms")
        for ln in _poly_expr(terms, T):
            A("      " + ln)
        A(f"      acc{k} = fma(wv{s}, P, acc{k});")
        A("    }")
    A("    {")
    A(f"      TI* __restrict__ op = out + z * {O}ll;")
    _row_store(A, "      ", st, T, st.layout_out, st.nseg_out, "op", lambda k: f"acc{k}")
    A("    }")
    A("  }")
    A("}")
    A("")

    # ------------------------------------------------------------------ backward
    A("// rows are visited in the order of the CSR grouping by weight index (csr_perm may be null: already grouped)")
    A("template <bool NEED_DW, bool NEED_DX>")
    A(f"__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu({bwd_waves}))) bwd_kernel(")
    A(f"    const TI* __restrict__ w, const TI* __restrict__ x, const TI* __restrict__ g, TI* __restrict__ dw, TI* __restrict__ dx,")
    A(f"    {T}* __restrict__ part, const void* __restrict__ w_index, int idx64, const int64_t* __restrict__ csr_perm, int64_t batch) {{")
    A("  const int lane = threadIdx.x;")
    A(f"  const int ch = blockIdx.x % {nch}; const int64_t slot = blockIdx.x / {nch}; const int64_t nslots = gridDim.x / {nch};")
    A(lane_setup)
    if stage_decl:
        A(stage_decl)
    A("  const int64_t p0 = slot * batch / nslots, p1 = (slot + 1) * batch / nslots;")
    A("  if (p0 >= p1) return;")
    for s in w_used:
        A(f"  {T} q{s} = 0, wv{s} = 0;")
    A("  int64_t cur = -1, first = -1;")
    A("  auto flush = [&](bool last) {")
    A("    if (!NEED_DW || !active) return;")
    A("    if (cur != first && !last) {                                     // whole group inside this slot")
    A(f"      TI* dst = dw + cur * {W}ll;")
    for s in range(st.nseg_w):
        A(f"      io_st({f'q{s}' if s in w_used else f'{T}(0)'}, dst + {s * E} + uu);")
    A("    } else {")
    A("      // head (the group may have begun in an earlier slot) or tail (it may continue in the next one): a partial row")
    A(f"      {T}* dst = part + (slot * 2 + (cur == first ? 0 : 1)) * {W}ll;")
    for s in range(st.nseg_w):
        A(f"      dst[{s * E} + uu] = {f'q{s}' if s in w_used else '0'};")
    A("    }")
    A("  };")
    A("  for (int64_t p = p0; p < p1; ++p) {")
    A("    const int64_t z = csr_perm ? csr_perm[p] : p;")
    A("    const int64_t e = load_index(w_index, idx64, z);")
    A("    if (e != cur) {")
    A("      if (cur >= 0) flush(false);")
    A("      if (first < 0) first = e;")
    A("      cur = e;")
    A(f"      const TI* __restrict__ wp = w + e * {W}ll;")
    for s in w_used:
        A(f"      wv{s} = io_ld(wp + {s * E} + uu); q{s} = 0;")
    A("    }")
    A(f"    const TI* __restrict__ xp = x + z * {X}ll;")
    A(f"    const TI* __restrict__ gp = g + z * {O}ll;")
    _row_request(A, "    ", st, T, st.layout_x, x_read, "xp", "xr", True)
    _row_request(A, "    ", st, T, st.layout_out, range(st.nseg_out), "gp", "gr", True)
    _row_unpack(A, "    ", st, T, st.layout_x, x_read, "xr", "xv")
    _row_unpack(A, "    ", st, T, st.layout_out, range(st.nseg_out), "gr", "gv")
    for a, b in pairs:
        A(f"    const {T} pp_{a}_{b} = xv{a} * xv{b};")
    for a in x_used:
        A(f"    {T} dxa{a} = 0;")
    for (s, k), terms in groups:
        A(f"    {{  // w[{s}] -> out[{k}]")
        A("      if (NEED_DW) {")
        for ln in _poly_expr(terms, T):
            A("        " + ln)
        A(f"        q{s} = fma(gv{k}, P, q{s});")
        A("      }")
        A("      if (NEED_DX) {")
        A(f"        const {T} wg = wv{s} * gv{k};")
        # d/dx of sum c * monomial, accumulated per variable: dx[v] += wg * sum c * (monomial / x[v])
        per_var = defaultdict(list)
        for xs, c in terms:
            for pos, v in enumerate(xs):
                rest = xs[:pos] + xs[pos + 1:]
                per_var[v].append((rest, c))
        for v, lst in sorted(per_var.items()):
            merged = defaultdict(float)
            for rest, c in lst:
                merged[rest] += c
            expr = None
            for rest, c in sorted(merged.items()):
                if len(rest) == 0:
                    term = _lit(c, T)
                    expr = term if expr is None else f"({expr} + {term})"
                    continue
                m = f"xv{rest[0]}" if len(rest) == 1 else f"pp_{rest[0]}_{rest[1]}"
                expr = f"{_lit(c, T)} * {m}" if expr is None else f"fma({_lit(c, T)}, {m}, {expr})"
            A(f"        dxa{v} = fma(wg, {expr}, dxa{v});")
        A("      }")
        A("    }")
    A("    if (NEED_DX) {")
    A(f"      TI* __restrict__ dp = dx + z * {X}ll;")
    _row_store(A, "      ", st, T, st.layout_x, st.nseg_x, "dp", lambda a: f"dxa{a}" if a in x_used else f"{T}(0)")
    A("    }")
    A("  }")
    A("  flush(true);")
    A("}")
    A("")
    A("// dw[e] = head / tail partials of the slots that meet the index group e; groups stored directly by one slot are left")
    A("// alone, empty groups are zeroed.  Positions [a, b) of the grouped order hold exactly the rows of group e, so a slot")
    A("// [q0, q1) contributes its head partial when a <= q0 < b (e is its first group) and its tail partial when only its")
    A("// last position lies in [a, b).  One block = 64 weight columns x 16 slot lanes; the 16 partial sums are added in lane")
    A("// order (fixed, so the result does not change from run to run).")
    A(f"__global__ void __launch_bounds__(1024) fold_kernel(const {T}* __restrict__ part, TI* __restrict__ dw,")
    A("    const int64_t* __restrict__ csr_offsets, int64_t batch, int64_t nslots, int64_t row0) {")
    A(f"  __shared__ {T} s_acc[16][64];")
    A("  __shared__ int s_any[16];")
    A("  const int64_t e = row0 + blockIdx.y;")
    A("  const int jl = threadIdx.x & 63, sl = threadIdx.x >> 6;")
    A("  const int j = blockIdx.x * 64 + jl;")
    A(f"  const bool live = j < {W};")
    A("  const int64_t a = csr_offsets[e], b = csr_offsets[e + 1];")
    A(f"  if (a == b) {{ if (sl == 0 && live) io_st({T}(0), dw + e * {W}ll + j); return; }}")
    A("  // slots whose range [s * batch / nslots, (s + 1) * batch / nslots) meets [a, b)")
    A("  int64_t s_lo = a * nslots / batch, s_hi = (b - 1) * nslots / batch;")
    A("  while (s_lo > 0 && (s_lo * batch / nslots) > a) --s_lo;")
    A("  while ((s_lo + 1) * batch / nslots <= a) ++s_lo;")
    A("  while (s_hi + 1 < nslots && ((s_hi + 1) * batch / nslots) < b) ++s_hi;")
    A("  while (s_hi * batch / nslots >= b) --s_hi;")
    A(f"  {T} acc = 0; bool any = false;")
    A("  for (int64_t s = s_lo + sl; s <= s_hi; s += 16) {")
    A("    const int64_t q0 = s * batch / nslots, q1 = (s + 1) * batch / nslots;")
    A("    if (q0 >= q1) continue;")
    A("    int half = -1;")
    A("    if (q0 >= a && q0 < b) half = 0; else if (q1 - 1 >= a && q1 - 1 < b) half = 1;")
    A(f"    if (half >= 0) {{ any = true; if (live) acc += part[(s * 2 + half) * {W}ll + j]; }}")
    A("  }")
    A("  s_acc[sl][jl] = acc;")
    A("  if (jl == 0) s_any[sl] = any ? 1 : 0;")
    A("  __syncthreads();")
    A("  if (sl == 0 && live) {")
    A(f"    {T} total = 0; int seen = 0;")
    A("    for (int t = 0; t < 16; ++t) { total += s_acc[t][jl]; seen |= s_any[t]; }")
    A(f"    if (seen) io_st(total, dw + e * {W}ll + j);")
    A("  }")
    A("}")
    A("")
    A(f"""
static bool all_dtype(const cueq_u1d_buffer* b, int n) {{ return common_dtype(b, n) == {io_code}; }}

static int64_t slots_for(int64_t batch, int waves) {{
  int64_t n = wave_slots(waves) / {nch};
  if (n > batch) n = batch;
  return n < 1 ? 1 : n;
}}

// buffers: w, x | out
static int run_fwd(const SpecCall& c) {{
  const cueq_u1d_buffer* b = c.buffers;
  if (!all_dtype(b, 3)) return CUEQ_ERR_UNSUPPORTED;
  if (b[1].batch_dim != CUEQ_BATCH_BATCHED || b[2].batch_dim != CUEQ_BATCH_BATCHED) return CUEQ_ERR_UNSUPPORTED;
  if (c.batch == 0) return CUEQ_OK;
  const dim3 grid(static_cast<unsigned>(slots_for(c.batch, {fwd_waves}) * {nch})), t(64);
  const TI* w = static_cast<const TI*>(b[0].data);
  const TI* x = static_cast<const TI*>(b[1].data);
  TI* o = static_cast<TI*>(b[2].data);
  KernelTimer timer("{name}_fwd_{tag}", c.stream);
  if (b[0].batch_dim == CUEQ_BATCH_INDEXED)
    hipLaunchKernelGGL(fwd_kernel<1>, grid, t, 0, c.stream, w, x, o, b[0].index, b[0].index_is_64, c.batch);
  else if (b[0].batch_dim == CUEQ_BATCH_SHARED)
    hipLaunchKernelGGL(fwd_kernel<2>, grid, t, 0, c.stream, w, x, o, nullptr, 0, c.batch);
  else
    hipLaunchKernelGGL(fwd_kernel<0>, grid, t, 0, c.stream, w, x, o, nullptr, 0, c.batch);
  CUEQ_CHECK_HIP(hipGetLastError());
  return CUEQ_OK;
}}

// buffers: w, x, g | [dw] [dx]; the weight must be indexed and its gradient carry the CSR grouping of that index
template <bool NEED_DW, bool NEED_DX>
static int64_t bwd_workspace(const cueq_u1d_buffer* b, int64_t batch) {{
  return NEED_DW ? slots_for(batch, {bwd_waves}) * 2 * {W}ll * static_cast<int64_t>(sizeof({T})) : 0;
}}

template <bool NEED_DW, bool NEED_DX>
static int run_bwd(const SpecCall& c) {{
  const cueq_u1d_buffer* b = c.buffers;
  constexpr int n = 3 + (NEED_DW ? 1 : 0) + (NEED_DX ? 1 : 0);
  if (!all_dtype(b, n)) return CUEQ_ERR_UNSUPPORTED;
  if (b[0].batch_dim != CUEQ_BATCH_INDEXED || b[1].batch_dim != CUEQ_BATCH_BATCHED || b[2].batch_dim != CUEQ_BATCH_BATCHED)
    return CUEQ_ERR_UNSUPPORTED;
  const cueq_u1d_buffer* bdw = NEED_DW ? &b[3] : nullptr;
  const cueq_u1d_buffer* bdx = NEED_DX ? &b[NEED_DW ? 4 : 3] : nullptr;
  if (bdx && bdx->batch_dim != CUEQ_BATCH_BATCHED) return CUEQ_ERR_UNSUPPORTED;
  if (bdw && (bdw->batch_dim != CUEQ_BATCH_INDEXED || bdw->index != b[0].index || bdw->rows != b[0].rows || !bdw->csr_offsets))
    return CUEQ_ERR_UNSUPPORTED;
  const int64_t batch = c.batch;
  TI* dw = bdw ? static_cast<TI*>(bdw->data) : nullptr;
  if (batch == 0) {{
    if (bdw && bdw->rows > 0) {{
      const int64_t nn = bdw->rows * {W}ll;
      hipLaunchKernelGGL(fill_zero<TI>, dim3(fill_blocks<TI>(nn)), dim3(256), 0, c.stream, dw, nn);
      CUEQ_CHECK_HIP(hipGetLastError());
    }}
    return CUEQ_OK;
  }}
  const int64_t nslots = slots_for(batch, {bwd_waves});
  const int64_t need = bwd_workspace<NEED_DW, NEED_DX>(b, batch);
  CUEQ_REQUIRE(need == 0 || (c.workspace && c.workspace_bytes >= need), CUEQ_ERR_INVALID, "workspace too small: need %lld bytes", (long long)need);
  {T}* part = static_cast<{T}*>(c.workspace);
  const int64_t* perm = bdw ? bdw->csr_perm : nullptr;
  {{
    KernelTimer timer("{name}_bwd_{tag}", c.stream);
    hipLaunchKernelGGL((bwd_kernel<NEED_DW, NEED_DX>), dim3(static_cast<unsigned>(nslots * {nch})), dim3(64), 0, c.stream,
                       static_cast<const TI*>(b[0].data), static_cast<const TI*>(b[1].data), static_cast<const TI*>(b[2].data), dw,
                       bdx ? static_cast<TI*>(bdx->data) : nullptr, part, b[0].index, b[0].index_is_64, perm, batch);
  }}
  CUEQ_CHECK_HIP(hipGetLastError());
  if (NEED_DW) {{
    // (the grid's y extent is the number of weight rows: at most 65535 of them per launch)
    for (int64_t r0 = 0; r0 < bdw->rows; r0 += 65535) {{
      const int64_t nr = bdw->rows - r0 < 65535 ? bdw->rows - r0 : 65535;
      hipLaunchKernelGGL(fold_kernel, dim3(({W} + 63) / 64, static_cast<unsigned>(nr)), dim3(1024), 0, c.stream, part, dw, bdw->csr_offsets,
                         batch, nslots, r0);
    }}
    CUEQ_CHECK_HIP(hipGetLastError());
  }}
  return CUEQ_OK;
}}

static const U1dSpec spec_fwd = {{0x{fwd_hash:016x}ull, "{name}_fwd_{tag}", run_fwd, nullptr, {io_code}}};
static SpecRegistrar reg_fwd(&spec_fwd);""")
    for (ndw, ndx), h in sorted(bwd_hashes.items()):
        which = ("w" if ndw else "") + ("x" if ndx else "")
        tb = f"<{str(ndw).lower()}, {str(ndx).lower()}>"
        A(f'static const U1dSpec spec_bwd_{which} = {{0x{h:016x}ull, "{name}_bwd_{which}_{tag}", run_bwd{tb}, bwd_workspace{tb}, {io_code}}};')
        A(f"static SpecRegistrar reg_bwd_{which}(&spec_bwd_{which});")
    A("")
    A(f"}}  // namespace {ns}")
    A("}  // namespace cueq")
    return "\n".join(L) + "\n"
