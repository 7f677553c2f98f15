"""Dense executor (``method="fused_tp"``): Linear and fully-connected tensor products on the matrix cores.

Mirror of ``cuequivariance_torch/cuequivariance_torch/primitives/segmented_polynomial_fused_tp.py:75-262``
for the polynomial forms the high-level layers produce:

* 3 operands ``weights[uv], x[iu] -> out[iv]``          (equivariant Linear, ``descriptors/irreps_tp.py:505-521``)
* 4 operands ``weights[uvw], x1[iu], x2[jv] -> out[kw]`` with ``v = 1`` (fully-connected product whose second
  operand has multiplicity one, e.g. spherical harmonics; ``descriptors/irreps_tp.py:22-47``)

with weights shared over the batch.  After the Clebsch-Gordan modes are flattened every path is a small
GEMM ``out[:, k_seg] += c * x2[:, j] * x1[:, i_seg] @ W_p``.  In float32 / bfloat16 the weight contractions run as a
few batched launches of the 128 x 128 tiled kernel (``cueq_gemm``, ``cueq_gemm_tn``) and the scaling by ``x2`` and the
sums over paths as one element-wise kernel per result (``cueq_fc_combine``, ``cueq_fc_rowdot``); float64 and shapes
those kernels refuse go through ``cueq_seg_gemm`` / ``cueq_seg_outer`` / ``cueq_seg_rowdot``.  First-order gradients only.
"""

from __future__ import annotations

import ctypes as C
import json
import threading
from collections import OrderedDict
from typing import Dict, List, Optional

import torch
import torch.nn as nn

from .. import _lib, cue

__all__ = ["SegmentedPolynomialDense"]

_DTYPE_CODE = {torch.float32: _lib.F32, torch.float64: _lib.F64, torch.bfloat16: _lib.BF16, torch.float16: _lib.F16}
_MATRIX_CORE = (torch.float32, torch.bfloat16, torch.float16)  # element types of the matrix-core kernels (float32 accumulation)
_FC_ELEMENT = {torch.float32: "float", torch.bfloat16: "uint16_t", torch.float16: "f16bits"}  # their names in the generated units


class _Path:
    __slots__ = ("w_off", "a_off", "j", "c_off", "K", "N", "coeff")

    def __init__(self, w_off, a_off, j, c_off, K, N, coeff):
        self.w_off, self.a_off, self.j, self.c_off, self.K, self.N, self.coeff = w_off, a_off, j, c_off, K, N, coeff


def _analyse(polynomial: cue.SegmentedPolynomial):
    """Flatten to per-path GEMMs.  Returns (paths, has_x2)."""
    if polynomial.num_outputs != 1 or len(polynomial.operations) != 1:
        raise NotImplementedError("fused_tp: exactly one operation with one output is supported")
    ope, stp = polynomial.operations[0]
    if tuple(ope.buffers) != tuple(range(stp.num_operands)) or stp.num_operands not in (3, 4):
        raise NotImplementedError(f"fused_tp supports 3 or 4 operands in buffer order. Got {stp.subscripts}.")
    if stp.num_paths == 0:
        raise NotImplementedError("fused_tp does not support empty paths.")
    # every mode that does not index the weights (the irrep components i, j, k) is flattened away
    try:
        d = stp.flatten_modes([m for m in stp.subscripts.modes() if m not in stp.subscripts.operands[0]])
    except ValueError as e:
        raise NotImplementedError(f"fused_tp does not support {stp.subscripts} (the weights come first): {e}") from e
    ss = d.subscripts.operands
    if stp.num_operands == 3:
        if not (len(ss[0]) == 2 and ss[1] == ss[0][0] and ss[2] == ss[0][1]):
            raise NotImplementedError(f"fused_tp does not support {d.subscripts} (expected uv,u,v)")
    else:
        # (uw,u,,w is the same contraction with the mode of extent one left out: the second operand is one scalar per segment)
        squeezed = len(ss[0]) == 2 and ss[1] == ss[0][0] and ss[2] == "" and ss[3] == ss[0][1]
        if not squeezed and not (len(ss[0]) == 3 and ss[1] == ss[0][0] and ss[2] == ss[0][1] and ss[3] == ss[0][2]):
            raise NotImplementedError(f"fused_tp does not support {d.subscripts} (expected uvw,u,v,w)")
        if not squeezed and d.get_dims(ss[2]) - {1}:
            raise NotImplementedError(
                "fused_tp: the second operand of a 4-operand contraction must have multiplicity 1 "
                f"(got extents {sorted(d.get_dims(ss[2]))})"
            )
    offs = [o.segment_offsets() for o in d.operands]
    paths = []
    for p in d.paths:
        c = float(p.coefficients)
        if c == 0.0:
            continue
        wshape = d.operands[0][p.indices[0]]
        K, N = wshape[0], wshape[-1]
        j = offs[2][p.indices[2]] if stp.num_operands == 4 else -1
        paths.append(_Path(offs[0][p.indices[0]], offs[1][p.indices[1]], j, offs[-1][p.indices[-1]], K, N, c))
    return paths, stp.num_operands == 4


def _problem_array(items):
    arr = (_lib.GemmProblem * max(1, len(items)))()
    for n, (a_off, c_off, b_off, s_col, trans_b, alpha, acc) in enumerate(items):
        arr[n].a_off, arr[n].c_off, arr[n].b_off = a_off, c_off, b_off
        arr[n].s_col, arr[n].trans_b, arr[n].alpha, arr[n].accumulate = s_col, trans_b, alpha, acc
    return arr


def _plan_gemm_launches(items_by_shape):
    """[(K, N, [problem tuples with the accumulate flag], aligned)]: problems of a launch write disjoint segments."""
    launches, written = [], set()
    for (K, N), items in items_by_shape.items():
        pending = list(items)
        while pending:
            launch, rest, seen = [], [], set()
            for it in pending:
                if it[1] in seen:
                    rest.append(it)
                else:
                    seen.add(it[1])
                    launch.append(it + (1 if it[1] in written else 0,))
            written |= seen
            launches.append((K, N, launch, all(it[0] % 8 == 0 for it in launch)))
            pending = rest
    return launches


class _DeviceTables:
    """Problem tables of one module uploaded to one device (read by the kernels with scalar loads)."""

    def __init__(self, mod: "SegmentedPolynomialDense", device: torch.device):
        def upload(ctypes_array):
            raw = bytes(ctypes_array)
            return torch.frombuffer(bytearray(raw), dtype=torch.uint8).to(device)

        self.fwd = [(K, N, upload(_problem_array(items)), len(items), ok) for K, N, items, ok in mod.fwd_launches]
        self.dx1 = [(K, N, upload(_problem_array(items)), len(items), ok) for K, N, items, ok in mod.dx1_launches]
        self.dw = []
        for (w_off, K, N), plist in mod.dw_groups.items():
            ent = (_lib.OuterEntry * len(plist))()
            for n, p in enumerate(plist):
                ent[n].a_off, ent[n].c_off, ent[n].s_col, ent[n].alpha = p.a_off, p.c_off, p.j, p.coeff
            self.dw.append((w_off, K, N, upload(ent), len(plist)))


def _run_gemms(dtype, A, B, S, Cout, launches):
    lib = _lib.load()
    stream = torch.cuda.current_stream(A.device).cuda_stream
    for K, N, table, n, aligned in launches:
        force_simple = 0 if (aligned and A.stride(0) % 8 == 0) else 1
        _lib.check(
            lib.cueq_seg_gemm(
                _DTYPE_CODE[dtype], K, N, A.data_ptr(), A.stride(0), B.data_ptr(),
                S.data_ptr() if S is not None else None, S.stride(0) if S is not None else 0,
                Cout.data_ptr(), Cout.stride(0), A.shape[0], table.data_ptr(), n, force_simple, stream,
            ),
            "cueq_seg_gemm",
        )


def _batched_groups(paths, a_key, c_key):
    """Group paths that share the weight block and scale into launches whose operand / result column offsets advance
    by constant strides: [(first path, count, stride of a, stride of c)]."""
    by_block: Dict[tuple, list] = {}
    for p in paths:
        by_block.setdefault((p.w_off, p.K, p.N, p.coeff), []).append(p)
    groups = []
    for plist in by_block.values():
        plist = sorted(plist, key=a_key)
        n = len(plist)
        da = a_key(plist[1]) - a_key(plist[0]) if n > 1 else 0
        dc = c_key(plist[1]) - c_key(plist[0]) if n > 1 else 0
        regular = n > 1 and da > 0 and dc > 0 and all(
            a_key(plist[t + 1]) - a_key(plist[t]) == da and c_key(plist[t + 1]) - c_key(plist[t]) == dc for t in range(n - 1)
        )
        if regular:
            groups.append((plist[0], n, da, dc))
        else:
            groups += [(q, 1, 0, 0) for q in plist]
    return groups


def _merged_weight_gradient(mod: "SegmentedPolynomialDense"):
    """``(K, N, coeff, a0, c0, da, dc, [(w_off, components)])`` when the weight gradients of all blocks of the 3-operand form
    can come from one launch: one block shape and scale, every weight block used by one run of components, and the
    components of all blocks at constant strides in the input and in the cotangent (a Linear layer over ``ir_mul`` rows:
    the components of all irreps one after the other).  ``None`` otherwise (one launch per block then)."""
    hit = getattr(mod, "_dw_merged", False)
    if hit is not False:
        return hit
    out = None
    comps = sorted(((p.a_off + i * da, p.c_off + i * dc, p.w_off, p.K, p.N, p.coeff) for p, count, da, dc in mod.fwd_groups
                    for i in range(count)))
    if len(comps) > 1 and len({c[3:] for c in comps}) == 1:
        K, N, coeff = comps[0][3:]
        da, dc = comps[1][0] - comps[0][0], comps[1][1] - comps[0][1]
        regular = da > 0 and dc > 0 and all(b[0] - a[0] == da and b[1] - a[1] == dc for a, b in zip(comps, comps[1:]))
        runs = []
        for c in comps:
            if runs and runs[-1][0] == c[2]:
                runs[-1][1] += 1
            else:
                runs.append([c[2], 1])
        if regular and len({w for w, _ in runs}) == len(runs) and len(comps) <= 64:
            out = (K, N, coeff, comps[0][0], comps[0][1], da, dc, [(w, n) for w, n in runs])
    mod._dw_merged = out
    return out


def _merged_tables(mod: "SegmentedPolynomialDense", device: torch.device):
    """For the 3-operand form: the column blocks of all paths as parts of table-driven launches, one launch per distinct
    (K, N, coefficient).  ``fwd``: rows (x offset, weight offset, out offset); ``dx``: rows (g offset, weight offset, dx
    offset); ``None`` when two parts of one launch would write the same columns (those take the per-group launches)."""
    key = (device.type, device.index)
    hit = mod._merged.get(key)
    if hit is None:
        by = {}
        for p in mod.paths:
            by.setdefault((p.K, p.N, p.coeff), []).append(p)
        ok = all(len({p.c_off for p in plist}) == len(plist) and len({p.a_off for p in plist}) == len(plist) for plist in by.values())
        outs = [p.c_off for p in mod.paths]
        ins = [p.a_off for p in mod.paths]
        ok = ok and len(set(outs)) == len(outs) and len(set(ins)) == len(ins)
        # the table-driven launch moves 16-byte vectors: extents and offsets in multiples of 8 elements
        ok = ok and all(v % 8 == 0 for p in mod.paths for v in (p.K, p.N, p.a_off, p.c_off, p.w_off))
        hit = None
        if ok:
            hit = [(K, N, coeff,
                    torch.tensor([(p.a_off, p.w_off, p.c_off) for p in plist], dtype=torch.int64, device=device),
                    torch.tensor([(p.c_off, p.w_off, p.a_off) for p in plist], dtype=torch.int64, device=device),
                    _rows_tables(K, N, plist))
                   for (K, N, coeff), plist in by.items()]
        mod._merged[key] = hit if hit is not None else False
        return hit
    return hit or None


def _rows_tables(K: int, N: int, plist):
    """Host tables for the row-streaming launch (``cueq_linear_rows``: every distinct weight block of a launch resident in
    the local data share): per element size a list of launches ``(forward table, input-gradient table, parts)``, the parts
    dealt out so that the weight blocks of one launch fit - or ``None`` where the launch's limits do not hold."""
    if K not in (32, 64, 96, 128) or N not in (32, 64, 96, 128):
        return None
    flat = lambda rows: (C.c_int64 * (3 * len(rows)))(*[v for r in rows for v in r])
    out = {}
    for es in (2, 4):
        room = 160 * 1024 - 8 * 32 * 144  # what the staging tiles of the eight wavefronts leave
        per_block = max(N * (es * K + 16), K * (es * N + 16))  # forward / input gradient
        cap = min(8, room // per_block)
        if cap < 1:
            return None
        groups, blocks = [], {}
        for p in plist:  # parts of one weight block stay together
            blocks.setdefault(p.w_off, []).append(p)
        cur = []
        for w_off, ps in blocks.items():
            if cur and (len({q.w_off for q in cur}) + 1 > cap or len(cur) + len(ps) > 48):
                groups.append(cur)
                cur = []
            cur = cur + ps
            while len(cur) > 48:
                groups.append(cur[:48])
                cur = cur[48:]
        if cur:
            groups.append(cur)
        out[es] = [(flat([(p.a_off, p.w_off, p.c_off) for p in g]), flat([(p.c_off, p.w_off, p.a_off) for p in g]), len(g)) for g in groups]
    return out


class _MulIrPlan:
    """Host tables of the 3-operand form on rows that keep the irrep component contiguous (``mul_ir``): every block
    ``(mul, ir)`` of the input is one part ``(a0, c0, w_off, K, N, d)`` - ``K * d`` consecutive elements of an input row,
    element (channel u, component i) at ``u * d + i``, ``N * d`` of an output row - served by ``cueq_linear_rows`` (d = 1: the
    block is the same in both layouts), ``cueq_linear_rows_mul_ir`` (d = 3, 5, 7) and ``cueq_linear_dw_mul_ir``.  ``None`` from
    ``build`` when the blocks are not of that shape."""

    def __init__(self, blocks):
        self.blocks = blocks
        self._tables: dict = {}

    @staticmethod
    def build(mod: "SegmentedPolynomialDense"):
        if mod.has_x2 or not mod.fwd_covers_output or not mod.dx1_covers_input:
            return None
        blocks = []
        for p, count, da, dc in mod.fwd_groups:  # the components of a block: `count` paths at strides (K, N)
            if count > 1 and (da != p.K or dc != p.N):
                return None
            if count not in (1, 3, 5, 7) or p.K % 32 or p.N % 32 or not (32 <= p.K <= 128 and 32 <= p.N <= 128):
                return None
            blocks.append((p.a_off, p.c_off, p.w_off, p.K, p.N, count, p.coeff))
        if len({b[2] for b in blocks}) != len(blocks) or not any(b[5] > 1 for b in blocks):
            return None  # (a weight block met twice is summed by the other path; nothing to gain without d > 1)
        if any(v % 8 for b in blocks for v in b[:3]):
            return None
        return _MulIrPlan(blocks)

    def accepts(self, dtype) -> bool:
        if dtype not in _MATRIX_CORE:
            return False
        us = 32 if dtype == torch.float32 else 64  # channels per slice of the row-streaming launch
        return all(d == 1 or (K % us == 0 and N % us == 0) for _, _, _, K, N, d, _ in self.blocks)

    def tables(self, es: int):
        """``(forward launches, input-gradient launches, weight-gradient launches)`` for elements of ``es`` bytes.
        forward / input gradient: ``(d, columns of the result block, contraction, table of (a, w, c[, d]), parts, coefficient)``;
        weight gradient: ``(K, N, coefficient, table, parts, [weight offset per part])``."""
        hit = self._tables.get(es)
        if hit is not None:
            return hit
        flat = lambda rows: (C.c_int64 * (len(rows[0]) * len(rows)))(*[v for r in rows for v in r])

        def fits(part, n_res, k_con):
            """What ``cueq_linear_rows_mul_ir`` checks: the weight blocks of the largest group of equal d and the staging
            tiles of the wavefronts within 160 KiB, at most 8 distinct blocks and 48 parts."""
            dmax = max(3, max(b[5] for b in part))
            waves = 8 if dmax * n_res <= 384 else 4
            slots = max(sum(1 for b in part if b[5] == d) for d in {b[5] for b in part})
            return (len(part) <= 8 and slots * n_res * (es * k_con + 16) + waves * 16 * (128 * dmax + 16) <= 160 * 1024)

        def launches(key, row):
            # One launch per number of components: the kernels are bound by what one compute unit keeps in flight, not
            # by the memory system, so the blocks of different d gain nothing from sharing a launch (measured: the three
            # blocks of 128x0e+128x1o+128x2e in one launch 265 us, in three 200 us) - and blocks of one component are the
            # same in both layouts and take the launch with 32-row units.
            by = {}
            for b in self.blocks:
                by.setdefault((b[5],) + key(b), []).append(b)
            out = []
            for (d, n_res, k_con, coeff), bl in by.items():
                if d == 1:
                    cap = max(1, min(8, (160 * 1024 - 8 * 32 * 144) // (n_res * (es * k_con + 16))))
                    for i in range(0, len(bl), cap):
                        part = bl[i: i + cap]
                        out.append((1, n_res, k_con, flat([row(q)[:3] for q in part]), len(part), coeff))
                    continue
                cur = []
                for b in bl:
                    if cur and not fits(cur + [b], n_res, k_con):
                        out.append((d, n_res, k_con, flat([row(q) for q in cur]), len(cur), coeff))
                        cur = []
                    cur.append(b)
                out.append((d, n_res, k_con, flat([row(q) for q in cur]), len(cur), coeff))
            return out

        fwd = launches(lambda b: (b[4], b[3], b[6]), lambda b: (b[0], b[2], b[1], b[5]))
        dx = launches(lambda b: (b[3], b[4], b[6]), lambda b: (b[1], b[2], b[0], b[5]))
        by = {}
        for b in self.blocks:
            by.setdefault((b[3], b[4], b[6]), []).append(b)
        dw = []
        for (K, N, coeff), bl in by.items():
            for i in range(0, len(bl), 32):
                part = bl[i: i + 32]
                dw.append((K, N, coeff, flat([(b[0], b[1], b[5]) for b in part]), len(part), [b[2] for b in part]))
        self._tables[es] = (fwd, dx, dw)
        return self._tables[es]


def _run_mul_ir(dtype, A, W, Cout, launches, forward: bool):
    """Forward (``W`` blocks ``K x N`` as they lie) or input gradient (the same blocks read as ``N x K``) of the ``mul_ir``
    parts: ``Cout[z, c0 + v d + i] = coeff * sum_u A[z, a0 + u d + i] W[u, v]``."""
    lib = _lib.load()
    stream = torch.cuda.current_stream(A.device).cuda_stream
    code = _DTYPE_CODE[dtype]
    for d, n_res, k_con, table, nparts, coeff in launches:
        if d == 1:
            _lib.check(lib.cueq_linear_rows(code, 1 if forward else 0, A.shape[0], n_res, k_con, A.data_ptr(), A.stride(0), W.data_ptr(), W.numel(),
                                            Cout.data_ptr(), Cout.stride(0), table, nparts, coeff, stream), "cueq_linear_rows")
        else:
            _lib.check(lib.cueq_linear_rows_mul_ir(code, 1 if forward else 0, A.shape[0], n_res, k_con, A.data_ptr(), A.stride(0), W.data_ptr(),
                                                   W.numel(), Cout.data_ptr(), Cout.stride(0), table, nparts, coeff, stream),
                       "cueq_linear_rows_mul_ir")


def _weight_gradient_mul_ir(dtype, x, g, numel, launches):
    """``dW`` (float32, flat) of the ``mul_ir`` parts: chunked partial products, then one ordered row sum per block."""
    lib = _lib.load()
    stream = torch.cuda.current_stream(x.device).cuda_stream
    code = _DTYPE_CODE[dtype]
    gw32 = torch.zeros(numel, dtype=torch.float32, device=x.device)
    for K, N, coeff, table, nparts, w_offs in launches:
        first = (C.c_int32 * (nparts + 1))()
        items = lib.cueq_linear_dw_mul_ir_items(x.shape[0], table, nparts, first)
        part = torch.empty(items, K * N, dtype=torch.float32, device=x.device)
        _lib.check(lib.cueq_linear_dw_mul_ir(code, K, N, x.shape[0], x.data_ptr(), x.stride(0), g.data_ptr(), g.stride(0), table, nparts,
                                             part.data_ptr(), coeff, stream), "cueq_linear_dw_mul_ir")
        ws_bytes = max(lib.cueq_sum_rows_workspace(first[p + 1] - first[p], K * N) for p in range(nparts))
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=x.device)
        for p, w_off in enumerate(w_offs):
            rows = part[first[p]: first[p + 1]]
            _lib.check(lib.cueq_sum_rows(_lib.F32, rows.shape[0], K * N, rows.data_ptr(), gw32[w_off: w_off + K * N].data_ptr(), ws.data_ptr(),
                                         ws_bytes, stream), "cueq_sum_rows")
    return gw32


def _vector_rows(*tensors) -> bool:
    return all(t.data_ptr() % 16 == 0 and (t.dim() < 2 or (t.stride(0) * t.element_size()) % 16 == 0) for t in tensors)


def _run_merged(dtype, A, B, Cout, launches, forward: bool):
    """``Cout[:, c : c + N] = coeff * A[:, a : a + K] @ W_p`` (forward, W_p is K x N as it lies) or
    ``Cout[:, a : a + K] = coeff * A[:, c : c + N] @ W_p^T`` (input gradient) for all parts of a launch at once."""
    lib = _lib.load()
    stream = torch.cuda.current_stream(A.device).cuda_stream
    code = _DTYPE_CODE[dtype]
    for K, N, coeff, fwd_tab, dx_tab, rows in launches:
        if rows is not None and dtype in _MATRIX_CORE:
            for fwd_host, dx_host, nparts in rows[A.element_size()]:
                if forward:
                    _lib.check(lib.cueq_linear_rows(code, 1, A.shape[0], N, K, A.data_ptr(), A.stride(0), B.data_ptr(), B.numel(), Cout.data_ptr(),
                                                    Cout.stride(0), fwd_host, nparts, coeff, stream), "cueq_linear_rows")
                else:
                    _lib.check(lib.cueq_linear_rows(code, 0, A.shape[0], K, N, A.data_ptr(), A.stride(0), B.data_ptr(), B.numel(), Cout.data_ptr(),
                                                    Cout.stride(0), dx_host, nparts, coeff, stream), "cueq_linear_rows")
        elif forward:
            _lib.check(lib.cueq_gemm_table(code, code, 0, 1, A.shape[0], N, K, A.data_ptr(), A.stride(0), B.data_ptr(), N,
                                           Cout.data_ptr(), Cout.stride(0), fwd_tab.data_ptr(), fwd_tab.shape[0], 1, 0, coeff, 0, stream),
                       "cueq_gemm_table")
        else:
            _lib.check(lib.cueq_gemm_table(code, code, 0, 0, A.shape[0], K, N, A.data_ptr(), A.stride(0), B.data_ptr(), N,
                                           Cout.data_ptr(), Cout.stride(0), dx_tab.data_ptr(), dx_tab.shape[0], 1, 0, coeff, 0, stream),
                       "cueq_gemm_table")


def _run_tiled(dtype, A, a_key, B_of, Cout, c_key, groups, Kdim, Ndim):
    """``Cout[:, c : c + N] (+)= coeff * A[:, a : a + K] @ B^T`` per group through the 128 x 128 tiled MFMA kernel
    (``cueq_gemm_nt``; ``B_of(path)`` gives the pointer of the ``N x K`` block)."""
    lib = _lib.load()
    stream = torch.cuda.current_stream(A.device).cuda_stream
    code = _DTYPE_CODE[dtype]
    es = A.element_size()
    written = set()
    for p, count, da, dc in groups:
        cols = tuple(c_key(p) + t * dc for t in range(count))
        acc = 1 if any(c in written for c in cols) else 0
        if acc and count > 1 and not all(c in written for c in cols):
            raise NotImplementedError("fused_tp: irregular overlap of output segments")
        written.update(cols)
        _lib.check(
            lib.cueq_gemm_nt(code, code, A.shape[0], Ndim(p), Kdim(p), A.data_ptr() + a_key(p) * es, A.stride(0), da,
                             B_of(p), Kdim(p), 0, Cout.data_ptr() + c_key(p) * es, Cout.stride(0), dc, count, p.coeff, acc,
                             stream),
            "cueq_gemm_nt",
        )
    return written


class _DenseFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, mod: "SegmentedPolynomialDense", w, x1, x2):
        dtype = x1.dtype
        Z = x1.shape[0]
        out = (torch.empty if mod.fwd_covers_output else torch.zeros)((Z, mod.out_size), dtype=dtype, device=x1.device)
        wd = w.detach().to(dtype).contiguous()
        x1d = x1.detach().contiguous()
        x2d = x2.detach().contiguous() if x2 is not None else None
        if Z > 0 and mod.rows_mul_ir:
            x1d, wd = _aligned(x1d), _aligned(wd)
            with torch.cuda.device(x1.device):
                _run_mul_ir(dtype, x1d, wd, out, mod.mul_ir.tables(x1d.element_size())[0], True)
        elif Z > 0:
            with torch.cuda.device(x1.device):
                merged = _merged_tables(mod, x1.device) if (mod.tiled(dtype, x1d, out) and _vector_rows(x1d, wd, out)) else None
                if merged is not None:
                    _run_merged(dtype, x1d, wd, out, merged, True)
                elif mod.tiled(dtype, x1d, out):
                    # out[:, k_seg] (+)= c * x1[:, i_seg] @ W_p: the kernel wants W_p^T (N x K, contraction contiguous)
                    wt = mod.transposed_weights(wd)
                    es = wd.element_size()
                    _run_tiled(dtype, x1d, lambda p: p.a_off, lambda p: wt.data_ptr() + p.w_off * es, out, lambda p: p.c_off,
                               mod.fwd_groups, lambda p: p.K, lambda p: p.N)
                else:
                    _run_gemms(dtype, x1d, wd, x2d, out, mod.tables(x1.device).fwd)
        ctx.mod = mod
        ctx.save_for_backward(w, x1, x2 if x2 is not None else torch.empty(0))
        ctx.has_x2 = x2 is not None
        return out

    @staticmethod
    def backward(ctx, g):
        mod = ctx.mod
        w, x1, x2 = ctx.saved_tensors
        if not ctx.has_x2:
            # the two gradients are functions of their own, each differentiable in terms of the other two:
            # derivatives of any order (forces and their training) stay on these kernels
            gx1 = _LinearDx.apply(mod, g, w, x1.dtype) if ctx.needs_input_grad[2] else None
            gw = _LinearDw.apply(mod, x1, g, w) if ctx.needs_input_grad[1] else None
            return None, gw, gx1, None
        if not torch.is_grad_enabled():  # (a plain backward: one call for the three gradients)
            return (None, *_fc_grads(0, mod, w, x1, x2, g, *ctx.needs_input_grad[1:4]))
        gw = _FcDw.apply(mod, x1, x2, g, w, 0) if ctx.needs_input_grad[1] else None
        gx1 = _FcDx1.apply(mod, w, g, x2, x1, 0) if ctx.needs_input_grad[2] else None
        gx2 = _FcDx2.apply(mod, w, x1, g, x2, 0) if ctx.needs_input_grad[3] else None
        return None, gw, gx1, gx2

    @staticmethod
    def _backward_impl(ctx, g, needs_input_grad):
        mod = ctx.mod
        w, x1, x2 = ctx.saved_tensors
        x2 = x2 if ctx.has_x2 else None
        dtype = x1.dtype
        lib = _lib.load()
        g = g.contiguous()
        wd = w.detach().to(dtype).contiguous()
        x1d = x1.detach().contiguous()
        x2d = x2.detach().contiguous() if x2 is not None else None
        Z = x1.shape[0]
        gw = gx1 = gx2 = None
        with torch.cuda.device(x1.device):
            tables = mod.tables(x1.device)
            stream = torch.cuda.current_stream(x1.device).cuda_stream
            if needs_input_grad[2]:
                # dx1[:, i_seg] += c * x2[:, j] * g[:, k_seg] @ W_p^T
                gx1 = (torch.empty_like if mod.dx1_covers_input else torch.zeros_like)(x1d)
                if Z > 0 and mod.rows_mul_ir:
                    _run_mul_ir(dtype, _aligned(g), _aligned(wd), gx1, mod.mul_ir.tables(g.element_size())[1], False)
                elif Z > 0:
                    merged = _merged_tables(mod, x1.device) if (mod.tiled(dtype, g, gx1) and _vector_rows(g, wd, gx1)) else None
                    if merged is not None:
                        _run_merged(dtype, g, wd, gx1, merged, False)
                    elif mod.tiled(dtype, g, gx1):
                        # dx1[:, i_seg] (+)= c * g[:, k_seg] @ W_p^T: W_p (K x N) is already "N x K" for this product
                        es = wd.element_size()
                        _run_tiled(dtype, g, lambda p: p.c_off, lambda p: wd.data_ptr() + p.w_off * es, gx1, lambda p: p.a_off,
                                   mod.dx1_groups, lambda p: p.N, lambda p: p.K)
                    else:
                        _run_gemms(dtype, g, wd, x2d, gx1, tables.dx1)
            if needs_input_grad[1]:
                gwd = None
                if Z > 0 and mod.rows_mul_ir:
                    gwd = _weight_gradient_mul_ir(dtype, _aligned(x1d), _aligned(g), wd.numel(), mod.mul_ir.tables(x1d.element_size())[2]).view(wd.shape)
                elif Z > 0 and mod.tiled(dtype, x1d, g):
                    # dW_p[k][n] += c * sum_z x1[z, i_seg + k] g[z, k_seg + n]: chunked partial products, ordered sum
                    # straight into a float32 image of the weights (a block met a second time is added)
                    code, es = _DTYPE_CODE[dtype], x1d.element_size()
                    gw32 = torch.zeros(wd.numel(), dtype=torch.float32, device=x1.device)
                    written = set()
                    merged = _merged_weight_gradient(mod)
                    if merged is not None:
                        # every component of every block in one launch (the partial products of a block's components are
                        # consecutive rows of `part`), then one ordered row sum per block
                        K, N, coeff, a0, c0, da, dc, runs = merged
                        nparts = sum(n for _, n in runs)
                        items = lib.cueq_gemm_tn_items(Z, nparts)
                        chunks = items // nparts
                        part = torch.empty(items, K * N, dtype=torch.float32, device=x1.device)
                        _lib.check(
                            lib.cueq_gemm_tn(code, K, N, Z, x1d.data_ptr() + a0 * es, x1d.stride(0), da, g.data_ptr() + c0 * es,
                                             g.stride(0), dc, nparts, part.data_ptr(), coeff, stream), "cueq_gemm_tn")
                        first_part = 0
                        for w_off, n in runs:
                            rows = part[first_part * chunks: (first_part + n) * chunks]
                            ws_bytes = lib.cueq_sum_rows_workspace(n * chunks, K * N)
                            ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=x1.device)
                            _lib.check(lib.cueq_sum_rows(_lib.F32, n * chunks, K * N, rows.data_ptr(), gw32[w_off: w_off + K * N].data_ptr(),
                                                         ws.data_ptr(), ws_bytes, stream), "cueq_sum_rows")
                            first_part += n
                    for p, count, da, dc in (mod.fwd_groups if merged is None else []):
                        items = lib.cueq_gemm_tn_items(Z, count)
                        part = torch.empty(items, p.K * p.N, dtype=torch.float32, device=x1.device)
                        _lib.check(
                            lib.cueq_gemm_tn(code, p.K, p.N, Z, x1d.data_ptr() + p.a_off * es, x1d.stride(0), da,
                                             g.data_ptr() + p.c_off * es, g.stride(0), dc, count, part.data_ptr(), p.coeff, stream),
                            "cueq_gemm_tn",
                        )
                        first = p.w_off not in written
                        written.add(p.w_off)
                        total = gw32[p.w_off: p.w_off + p.K * p.N] if first else torch.empty(p.K * p.N, dtype=torch.float32, device=x1.device)
                        ws_bytes = lib.cueq_sum_rows_workspace(items, p.K * p.N)
                        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=x1.device)
                        _lib.check(lib.cueq_sum_rows(_lib.F32, items, p.K * p.N, part.data_ptr(), total.data_ptr(), ws.data_ptr(),
                                                     ws_bytes, stream), "cueq_sum_rows")
                        if not first:
                            gw32[p.w_off: p.w_off + p.K * p.N] += total
                    gwd = gw32.view(wd.shape)
                elif Z > 0:
                    gwd = torch.zeros_like(wd)
                    for w_off, K, N, ent, n in tables.dw:
                        ws_bytes = lib.cueq_seg_outer_workspace(_DTYPE_CODE[dtype], K, N, Z)
                        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x1.device)
                        _lib.check(
                            lib.cueq_seg_outer(
                                _DTYPE_CODE[dtype], K, N, x1d.data_ptr(), x1d.stride(0), g.data_ptr(), g.stride(0),
                                x2d.data_ptr() if x2d is not None else None, x2d.stride(0) if x2d is not None else 0,
                                gwd.data_ptr() + w_off * gwd.element_size(), Z, ent.data_ptr(), n, 0, 0,
                                ws.data_ptr(), ws_bytes, stream,
                            ),
                            "cueq_seg_outer",
                        )
                if gwd is None:
                    gwd = torch.zeros_like(wd)
                gw = gwd.to(w.dtype).reshape(w.shape)
            if x2 is not None and needs_input_grad[3]:
                gx2 = torch.zeros_like(x2d)
                touched = set()
                for p in mod.paths:
                    if Z == 0:
                        break
                    pr = _problem_array([(p.a_off, p.c_off, p.w_off, p.j, 0, p.coeff, 1 if p.j in touched else 0)])
                    touched.add(p.j)
                    _lib.check(
                        lib.cueq_seg_rowdot(
                            _DTYPE_CODE[dtype], p.K, p.N, x1d.data_ptr(), x1d.stride(0), wd.data_ptr(), g.data_ptr(),
                            g.stride(0), gx2.data_ptr(), gx2.stride(0), Z, pr, stream,
                        ),
                        "cueq_seg_rowdot",
                    )
        return None, gw, gx1, gx2


class _GradContext:
    """What ``_DenseFunction._backward_impl`` reads from an autograd context."""

    def __init__(self, mod, w, x1):
        self.mod, self.saved_tensors, self.has_x2 = mod, (w, x1, torch.empty(0)), False


class _LinearDx(torch.autograd.Function):
    """``dx = g W^T`` of the 3-operand form as a function of ``(g, w)``: linear in both, so its own gradients are the
    forward product (with respect to ``g``) and the weight-gradient product (with respect to ``w``)."""

    @staticmethod
    def forward(ctx, mod, g, w, x_dtype):
        x_like = torch.empty(g.shape[0], mod.input_sizes[1], dtype=x_dtype, device=g.device)
        gx1 = _DenseFunction._backward_impl(_GradContext(mod, w, x_like), g.to(x_dtype), (False, False, True, False))[2]
        ctx.mod = mod
        ctx.save_for_backward(g, w)
        return gx1

    @staticmethod
    def backward(ctx, c):
        g, w = ctx.saved_tensors
        dg = _DenseFunction.apply(ctx.mod, w, c, None).to(g.dtype) if ctx.needs_input_grad[1] else None
        dw = _LinearDw.apply(ctx.mod, c, g, w) if ctx.needs_input_grad[2] else None
        return None, dg, dw, None


class _LinearDw(torch.autograd.Function):
    """``dW = x^T g`` (per weight block, with the path coefficients) as a function of ``(x, g)``; ``w`` only gives the
    shape and dtype of the result."""

    @staticmethod
    def forward(ctx, mod, x1, g, w):
        gw = _DenseFunction._backward_impl(_GradContext(mod, w, x1), g.to(x1.dtype), (False, True, False, False))[1]
        ctx.mod = mod
        ctx.save_for_backward(x1, g)
        return gw

    @staticmethod
    def backward(ctx, c):
        x1, g = ctx.saved_tensors
        dx = _LinearDx.apply(ctx.mod, g, c, x1.dtype) if ctx.needs_input_grad[1] else None
        dg = _DenseFunction.apply(ctx.mod, c, x1, None).to(g.dtype) if ctx.needs_input_grad[2] else None
        return None, dx, dg, None


def _progressions(items, key_a, key_c):
    """Split ``items`` (sorted) into runs whose ``key_a`` and ``key_c`` advance by constant positive strides:
    ``[(first item, count, stride a, stride c)]`` - one batched GEMM launch each."""
    runs, i = [], 0
    while i < len(items):
        j = i + 1
        da = dc = 0
        if j < len(items):
            da, dc = key_a(items[j]) - key_a(items[i]), key_c(items[j]) - key_c(items[i])
            if da > 0 and dc > 0:
                while j + 1 < len(items) and key_a(items[j + 1]) - key_a(items[j]) == da and key_c(items[j + 1]) - key_c(items[j]) == dc:
                    j += 1
                j += 1
            else:
                da = dc = 0
        runs.append((items[i], j - i, da, dc))
        i = j
    return runs


class _FcPlan:
    """Host tables of the fully-connected product on the tiled GEMMs (see ``cueq_fc_combine`` in the header):
    ``T[:, t] = x1[:, i_seg] @ W_p`` per distinct (weight block, x1 segment), ``G[:, g] = g[:, k_seg] @ W_p^T`` per distinct
    (weight block, output segment); every flattened path is then one scaled use of a ``T`` (forward, ``H`` for the weight
    gradient) or of a ``G`` (``dx1``, ``dx2``)."""

    def __init__(self, paths, n2: int):
        import numpy as np

        self.n2 = n2
        t_of, g_of = {}, {}
        t_cols = g_cols = 0
        for p in sorted(paths, key=lambda p: (p.w_off, p.a_off)):
            if (p.w_off, p.a_off) not in t_of:
                t_of[(p.w_off, p.a_off)] = (t_cols, p.K, p.N)
                t_cols += p.N
        for p in sorted(paths, key=lambda p: (p.w_off, p.c_off)):
            if (p.w_off, p.c_off) not in g_of:
                g_of[(p.w_off, p.c_off)] = (g_cols, p.K, p.N)
                g_cols += p.K
        self.t_cols, self.g_cols = t_cols, g_cols
        # one table-driven GEMM launch per block shape: rows (operand offset, weight offset, result offset)
        self.t_shapes, self.g_shapes = {}, {}
        for (w_off, a_off), (t, K, N) in sorted(t_of.items()):
            self.t_shapes.setdefault((K, N), []).append((a_off, w_off, t))
        for (w_off, c_off), (gq, K, N) in sorted(g_of.items()):
            self.g_shapes.setdefault((K, N), []).append((c_off, w_off, gq))
        def tables(block_key, block_n, src):
            blocks = {}
            for p in paths:
                blocks.setdefault((block_key(p), block_n(p)), []).append((p.j, src(p), p.coeff))
            barr = np.zeros(len(blocks), dtype=[("off", "<i4"), ("n", "<i4"), ("first", "<i4"), ("num", "<i4")])
            uarr = np.zeros(sum(len(u) for u in blocks.values()), dtype=[("j", "<i4"), ("src", "<i4"), ("coeff", "<f4"), ("pad", "<i4")])
            first = 0
            for b, ((off, n), us) in enumerate(sorted(blocks.items())):
                barr[b] = (off, n, first, len(us))
                for u in us:
                    uarr[first] = (u[0], u[1], u[2], 0)
                    first += 1
            # (last entry: every block width and column offset is a multiple of four - four columns per thread)
            vec = all(off % 4 == 0 and n % 4 == 0 for off, n in blocks) and all(u[1] % 4 == 0 for us in blocks.values() for u in us)
            return barr, uarr, max(n for _, n in blocks), vec

        self.fwd = tables(lambda p: p.c_off, lambda p: p.N, lambda p: t_of[(p.w_off, p.a_off)][0])
        self.dx1 = tables(lambda p: p.a_off, lambda p: p.K, lambda p: g_of[(p.w_off, p.c_off)][0])
        self.h = tables(lambda p: t_of[(p.w_off, p.a_off)][0], lambda p: p.N, lambda p: p.c_off)
        darr = np.zeros(len(paths), dtype=[("j", "<i4"), ("a", "<i4"), ("g", "<i4"), ("k", "<i4"), ("coeff", "<f4"), ("pad", "<i4", 3)])
        for u, p in enumerate(sorted(paths, key=lambda p: p.j)):  # by column: uses of one column share a reduction
            darr[u] = (p.j, p.a_off, g_of[(p.w_off, p.c_off)][0], p.K, p.coeff, (0, 0, 0))
        self.dx2 = darr
        self.dx2_vec = all(v % 4 == 0 for p in paths for v in (p.K, p.a_off, g_of[(p.w_off, p.c_off)][0]))
        self.ok = max(self.fwd[2], self.dx1[2], self.h[2]) <= 256 and n2 <= 64
        self._device: Dict[int, dict] = {}

    def device(self, dev: torch.device) -> dict:
        idx = dev.index if dev.index is not None else torch.cuda.current_device()
        d = self._device.get(idx)
        if d is None:
            def up(a):
                return torch.from_numpy(a.view("u1").reshape(-1).copy()).to(torch.device("cuda", idx))

            device = torch.device("cuda", idx)
            t_tabs, g_tabs, w_tabs = {}, {}, {}
            for (K, N), rows in self.t_shapes.items():
                t_tabs[(K, N)] = torch.tensor(rows, dtype=torch.int64, device=device)
                # weight gradient: part p contracts x1[:, a_off_p : +K] with H[:, t_p : +N] into block p of the partials
                # the parts of one weight block (its x1 components) are summed in a fixed order: for every distinct
                # block the list of its parts, padded with the index of an all-zero extra part
                blocks = sorted({w for _, w, _ in rows})
                members = [[p for p, (_, w, _) in enumerate(rows) if w == wb] for wb in blocks]
                width = max(len(m) for m in members)
                w_tabs[(K, N)] = (
                    torch.tensor([(a, t, p * K * N) for p, (a, _, t) in enumerate(rows)], dtype=torch.int64, device=device),
                    torch.tensor([m + [len(rows)] * (width - len(m)) for m in members], dtype=torch.int64, device=device),
                    (torch.tensor(blocks, dtype=torch.int64, device=device)[:, None]
                     + torch.arange(K * N, dtype=torch.int64, device=device)[None, :]).reshape(-1),
                )
            for (K, N), rows in self.g_shapes.items():
                g_tabs[(K, N)] = torch.tensor(rows, dtype=torch.int64, device=device)
            d = self._device[idx] = {
                "t": t_tabs, "g": g_tabs, "w": w_tabs,
                "fwd": (up(self.fwd[0]), up(self.fwd[1]), len(self.fwd[0]), self.fwd[2], self.fwd[3]),
                "dx1": (up(self.dx1[0]), up(self.dx1[1]), len(self.dx1[0]), self.dx1[2], self.dx1[3]),
                "h": (up(self.h[0]), up(self.h[1]), len(self.h[0]), self.h[2], self.h[3]),
                "dx2": (up(self.dx2), len(self.dx2)),
            }
        return d


def _aligned(t: torch.Tensor) -> torch.Tensor:
    """``t`` contiguous and starting on a 16-byte boundary (a copy when a view starts elsewhere): the fully connected
    kernels move rows in 16-byte pieces."""
    t = t.contiguous()
    return t.clone() if t.data_ptr() % 16 else t


def _fc_combine(lib, code, t_code, Z, S, T, O, table, stream):
    blocks, uses, nblocks, max_n, vec = table
    _lib.check(lib.cueq_fc_combine(code, t_code, Z, S.data_ptr(), S.stride(0), T.data_ptr(), T.stride(0), O.data_ptr(), O.stride(0),
                                   blocks.data_ptr(), nblocks, uses.data_ptr(), max_n, 1 if vec else 0, stream), "cueq_fc_combine")


class _FcFunction(torch.autograd.Function):
    """Fully-connected product (shared weights, second operand of multiplicity one) on the tiled GEMMs: a few batched
    ``cueq_gemm`` launches for the weight contractions and one ``cueq_fc_combine`` / ``cueq_fc_rowdot`` per result."""

    @staticmethod
    def forward(ctx, mod: "SegmentedPolynomialDense", w, x1, x2):
        dtype, dev = x1.dtype, x1.device
        Z = x1.shape[0]
        plan, lib = mod.fc_plan, _lib.load()
        out = (torch.empty if mod.fwd_covers_output else torch.zeros)((Z, mod.out_size), dtype=dtype, device=dev)
        if Z > 0:
            wd, x1d, x2d = _aligned(w.detach().to(dtype)), _aligned(x1.detach()), x2.detach().contiguous()
            with torch.cuda.device(dev):
                stream = torch.cuda.current_stream(dev).cuda_stream
                code, es = _DTYPE_CODE[dtype], x1d.element_size()
                unit = mod.fused_unit(dtype, x1d, out)
                if unit is None and mod.rows_mul_ir:
                    raise NotImplementedError("fused_tp: rows='mul_ir' needs the generated fused kernels")
                if unit is not None:
                    if unit.fcj_fwd(Z, wd.data_ptr(), x1d.data_ptr(), x1d.stride(0), x2d.data_ptr(), x2d.stride(0), out.data_ptr(),
                                    out.stride(0), stream) != 0:
                        raise RuntimeError("fused fully connected forward: launch failed")
                    ctx.mod = mod
                    ctx.save_for_backward(w, x1, x2)
                    return out
                T = torch.empty(Z, plan.t_cols, dtype=torch.float32, device=dev)
                tables = plan.device(dev)
                for (K, N), tab in tables["t"].items():
                    # T[:, t : + N] = x1[:, a_off : + K] @ W_p for every row (a_off, w_off, t) of the table; W_p is K x N:
                    # contraction-major as it lies
                    _lib.check(lib.cueq_gemm_table(code, _lib.F32, 0, 1, Z, N, K, x1d.data_ptr(), x1d.stride(0), wd.data_ptr(), N,
                                                   T.data_ptr(), plan.t_cols, tab.data_ptr(), tab.shape[0], 1, 0, 1.0, 0, stream),
                               "cueq_gemm_table")
                _fc_combine(lib, code, _lib.F32, Z, x2d, T, out, tables["fwd"], stream)
        ctx.mod = mod
        ctx.save_for_backward(w, x1, x2)
        return out

    @staticmethod
    def backward(ctx, g):
        # each gradient is a function of its own, trilinear like the product and differentiable in terms of the other
        # three: derivatives of any order stay on these kernels
        mod = ctx.mod
        w, x1, x2 = ctx.saved_tensors
        if not torch.is_grad_enabled():
            # a plain backward (no graph of the gradients asked for): the three gradients in one call, their operands
            # prepared once
            return (None, *_fc_grads(1, mod, w, x1, x2, g, *ctx.needs_input_grad[1:4]))
        gw = _FcDw.apply(mod, x1, x2, g, w, 1) if ctx.needs_input_grad[1] else None
        gx1 = _FcDx1.apply(mod, w, g, x2, x1, 1) if ctx.needs_input_grad[2] else None
        gx2 = _FcDx2.apply(mod, w, x1, g, x2, 1) if ctx.needs_input_grad[3] else None
        return None, gw, gx1, gx2

    @staticmethod
    def grads(mod, w, x1, x2, g, need_w, need_x1, need_x2):
        """``(dw, dx1, dx2)`` (``None`` where not asked for) of the product for the cotangent ``g``."""
        dtype, dev = x1.dtype, x1.device
        Z = x1.shape[0]
        plan, lib = mod.fc_plan, _lib.load()
        g = _aligned(g.detach().to(dtype))
        wd, x1d, x2d = _aligned(w.detach().to(dtype)), _aligned(x1.detach()), x2.detach().to(dtype).contiguous()
        gw = gx1 = gx2 = None
        with torch.cuda.device(dev):
            stream = torch.cuda.current_stream(dev).cuda_stream
            code, es = _DTYPE_CODE[dtype], x1d.element_size()
            unit = unit_w = mod.fused_unit(dtype, x1d, g) if Z > 0 else None
            tables = plan.device(dev) if unit is None else None  # (the fused kernels carry their tables in their code)
            if unit is None and mod.rows_mul_ir and Z > 0:
                raise NotImplementedError("fused_tp: rows='mul_ir' needs the generated fused kernels")
            if need_x1:  # (the generated kernels write every column)
                gx1 = (torch.empty_like if mod.dx1_covers_input or unit is not None else torch.zeros_like)(x1d)
            if need_x2:
                gx2 = (torch.empty_like if unit is not None else torch.zeros_like)(x2d)
            both = -2
            if unit is not None and need_x1 and need_x2:  # one pass over the products g W^T serves both (-2: not for this product)
                part = torch.empty(Z, 2 * x2d.shape[1], dtype=torch.float32, device=dev)
                both = unit.fcj_dx12(Z, wd.data_ptr(), g.data_ptr(), g.stride(0), x2d.data_ptr(), x2d.stride(0), x1d.data_ptr(), x1d.stride(0),
                                     gx1.data_ptr(), gx1.stride(0), gx2.data_ptr(), gx2.stride(0), part.data_ptr(), stream)
                if both not in (0, -2):
                    raise RuntimeError("fused fully connected gradients (both operands): launch failed")
            if both == 0:
                pass
            elif unit is not None:
                if need_x1 and unit.fcj_dx1(Z, wd.data_ptr(), g.data_ptr(), g.stride(0), x2d.data_ptr(), x2d.stride(0), gx1.data_ptr(),
                                            gx1.stride(0), stream) != 0:
                    raise RuntimeError("fused fully connected gradient (first operand): launch failed")
                if need_x2 and unit.fcj_dx2(Z, wd.data_ptr(), x1d.data_ptr(), x1d.stride(0), x2d.data_ptr(), x2d.stride(0), g.data_ptr(),
                                            g.stride(0), gx2.data_ptr(), gx2.stride(0), stream) != 0:
                    raise RuntimeError("fused fully connected gradient (second operand): launch failed")
            elif (need_x1 or need_x2) and Z > 0:
                G = torch.empty(Z, plan.g_cols, dtype=torch.float32, device=dev)
                for (K, N), tab in tables["g"].items():
                    # G[:, gq : + K] = g[:, c_off : + N] @ W_p^T for every row (c_off, w_off, gq); W_p (K x N) is
                    # "rows x contraction" for this product
                    _lib.check(lib.cueq_gemm_table(code, _lib.F32, 0, 0, Z, K, N, g.data_ptr(), g.stride(0), wd.data_ptr(), N,
                                                   G.data_ptr(), plan.g_cols, tab.data_ptr(), tab.shape[0], 1, 0, 1.0, 0, stream),
                               "cueq_gemm_table")
                if need_x1:
                    _fc_combine(lib, code, _lib.F32, Z, x2d, G, gx1, tables["dx1"], stream)
                if need_x2:
                    uses, nuses = tables["dx2"]
                    _lib.check(lib.cueq_fc_rowdot(code, _lib.F32, Z, x1d.data_ptr(), x1d.stride(0), G.data_ptr(), plan.g_cols,
                                                  gx2.data_ptr(), gx2.stride(0), plan.n2, uses.data_ptr(), nuses,
                                                  1 if plan.dx2_vec else 0, stream), "cueq_fc_rowdot")
            if unit_w is not None and need_w:
                # per-block partial sums of the generated kernel (x1^T H with H formed in registers), then a row sum
                numel = wd.numel()
                shape = mod._dw_shapes.get((Z, dtype))  # (chunk count and row-sum workspace: two library calls per batch size)
                if shape is None:
                    nb = unit_w.fcj_dw_blocks(Z)
                    if len(mod._dw_shapes) >= 64:
                        mod._dw_shapes.clear()
                    shape = mod._dw_shapes[(Z, dtype)] = (nb, lib.cueq_sum_rows_workspace(nb, numel),
                                                          sum(K * N for _, K, N in mod.weight_blocks) == numel)
                nblocks, ws_bytes, covered = shape
                part = (torch.empty if covered else torch.zeros)(nblocks, numel, dtype=torch.float32, device=dev)
                if unit_w.fcj_dw(Z, x1d.data_ptr(), x1d.stride(0), x2d.data_ptr(), x2d.stride(0), g.data_ptr(), g.stride(0),
                                 part.data_ptr(), numel, stream) != 0:
                    raise RuntimeError("fused fully connected weight gradient: launch failed")
                gw32 = torch.empty(numel, dtype=torch.float32, device=dev)
                ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
                _lib.check(lib.cueq_sum_rows(_lib.F32, nblocks, numel, part.data_ptr(), gw32.data_ptr(), ws.data_ptr(), ws_bytes, stream),
                           "cueq_sum_rows")
                gw = gw32.to(w.dtype).reshape(w.shape)
            elif need_w:
                gwd = torch.zeros_like(wd)
                if Z > 0:
                    # H[:, t] = sum over the uses of T-block t of coeff * x2[:, j] * g[:, k_seg]; then dW_p = sum_i x1[:, i_seg]^T H[:, t_i]
                    H = torch.empty(Z, plan.t_cols, dtype=dtype, device=dev)
                    _fc_combine(lib, code, code, Z, x2d, g, H, tables["h"], stream)
                    gw32 = torch.zeros(wd.numel(), dtype=torch.float32, device=dev)
                    for (K, N), (tab, members, dst) in tables["w"].items():
                        nparts = tab.shape[0]
                        if K <= 64 and N <= 64:  # one wavefront per 64 x 64 product: about two of them per SIMD
                            chunks = max(1, min(-(-2048 // nparts), Z // 64))
                        else:
                            tiles = ((K + 127) // 128) * ((N + 127) // 128)
                            chunks = max(1, min(-(-512 // (nparts * tiles)), Z // 256))
                        part = torch.empty(chunks, nparts * K * N, dtype=torch.float32, device=dev)
                        _lib.check(lib.cueq_gemm_table(code, _lib.F32, 1, 1, K, N, Z, x1d.data_ptr(), x1d.stride(0), H.data_ptr(),
                                                       plan.t_cols, part.data_ptr(), N, tab.data_ptr(), nparts, chunks, nparts * K * N,
                                                       1.0, 0, stream), "cueq_gemm_table")
                        total = torch.zeros((nparts + 1) * K * N, dtype=torch.float32, device=dev)  # (+ the all-zero part)
                        ws_bytes = lib.cueq_sum_rows_workspace(chunks, nparts * K * N)
                        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
                        _lib.check(lib.cueq_sum_rows(_lib.F32, chunks, nparts * K * N, part.data_ptr(), total.data_ptr(), ws.data_ptr(),
                                                     ws_bytes, stream), "cueq_sum_rows")
                        # blocks of one path (its x1 components) land on the same weights: ordered sum, then a copy
                        # to distinct destinations (index_add_ would use atomics)
                        gw32.index_copy_(0, dst, total.view(nparts + 1, K * N)[members].sum(1).reshape(-1))
                    gwd = gw32.to(dtype).view(wd.shape)
                gw = gwd.to(w.dtype).reshape(w.shape)
            if gx2 is not None and x2.shape[0] == 1 and Z != 1:
                gx2 = gx2.sum(0, keepdim=True)
        return gw, gx1, gx2


def _fc_grads(kind, mod, w, x1, x2, g, need_w, need_x1, need_x2):
    """``(dw, dx1, dx2)`` of the 4-operand product: ``kind`` 1 on the fully connected kernels (float32 / bfloat16), 0 on
    the per-path kernels (float64, shapes the others do not take)."""
    if kind == 1:
        return _FcFunction.grads(mod, w, x1, x2, g, need_w, need_x1, need_x2)
    ctx = _GradContext(mod, w, x1)
    ctx.saved_tensors, ctx.has_x2 = (w, x1, x2), True
    return _DenseFunction._backward_impl(ctx, g.detach().to(x1.dtype), (False, need_w, need_x1, need_x2))[1:4]


class _FcDw(torch.autograd.Function):
    """``dW(x1, x2, g)``; ``w`` gives the shape and dtype of the result."""

    @staticmethod
    def forward(ctx, mod, x1, x2, g, w, kind):
        ctx.mod, ctx.kind = mod, kind
        ctx.save_for_backward(x1, x2, g)
        return _fc_grads(kind, mod, w, x1, x2, g, True, False, False)[0]

    @staticmethod
    def backward(ctx, c):  # c: shaped like the weights
        x1, x2, g = ctx.saved_tensors
        need = ctx.needs_input_grad
        return (None,
                _FcDx1.apply(ctx.mod, c, g, x2, x1, ctx.kind) if need[1] else None,
                _FcDx2.apply(ctx.mod, c, x1, g, x2, ctx.kind) if need[2] else None,
                _FUNCTIONS[ctx.kind].apply(ctx.mod, c, x1, x2).to(g.dtype) if need[3] else None,
                None, None)


class _FcDx1(torch.autograd.Function):
    """``dx1(w, g, x2)``; ``x1`` gives the dtype of the result."""

    @staticmethod
    def forward(ctx, mod, w, g, x2, x1, kind):
        ctx.mod, ctx.kind = mod, kind
        ctx.save_for_backward(w, g, x2)
        return _fc_grads(kind, mod, w, x1, x2, g, False, True, False)[1]

    @staticmethod
    def backward(ctx, c):  # c: shaped like x1
        w, g, x2 = ctx.saved_tensors
        need = ctx.needs_input_grad
        return (None,
                _FcDw.apply(ctx.mod, c, x2, g, w, ctx.kind) if need[1] else None,
                _FUNCTIONS[ctx.kind].apply(ctx.mod, w, c, x2).to(g.dtype) if need[2] else None,
                _FcDx2.apply(ctx.mod, w, c, g, x2, ctx.kind) if need[3] else None,
                None, None)


class _FcDx2(torch.autograd.Function):
    """``dx2(w, x1, g)``; ``x2`` gives the shape and dtype of the result."""

    @staticmethod
    def forward(ctx, mod, w, x1, g, x2, kind):
        ctx.mod, ctx.kind = mod, kind
        ctx.save_for_backward(w, x1, g)
        return _fc_grads(kind, mod, w, x1, x2, g, False, False, True)[2]

    @staticmethod
    def backward(ctx, c):  # c: shaped like x2
        w, x1, g = ctx.saved_tensors
        need = ctx.needs_input_grad
        return (None,
                _FcDw.apply(ctx.mod, x1, c, g, w, ctx.kind) if need[1] else None,
                _FcDx1.apply(ctx.mod, w, g, c, x1, ctx.kind) if need[2] else None,
                _FUNCTIONS[ctx.kind].apply(ctx.mod, w, x1, c).to(g.dtype) if need[3] else None,
                None, None)


def _row_ranges(Z: int, Cn: int, offsets: torch.Tensor):
    """Row ranges for the rows-grouped launches (``cueq_gemm_grouped`` mode 1 keeps its row tiles, one extra per class,
    on grid.y: 65 535 of them), each with the class offsets relative to the range - computed on the device, no
    synchronisation."""
    cap = (65535 - Cn - 1) * 128
    if Z <= cap:
        return [(0, Z, offsets)]
    return [(lo, min(Z, lo + cap), (offsets - lo).clamp_(0, min(Z, lo + cap) - lo)) for lo in range(0, Z, cap)]


class _IndexedDenseFunction(torch.autograd.Function):
    """Linear with one weight row per class and the batch rows sorted by class (``offsets[c] .. offsets[c+1]`` are the rows
    of class ``c``): grouped GEMMs on the tiled MFMA kernel (``cueq_gemm_grouped``), no host synchronisation."""

    @staticmethod
    def forward(ctx, mod: "SegmentedPolynomialDense", w, x1, offsets):
        dtype = x1.dtype
        Z, Cn, W = x1.shape[0], w.shape[0], w.shape[1]
        lib = _lib.load()
        out = (torch.empty if mod.fwd_covers_output else torch.zeros)((Z, mod.out_size), dtype=dtype, device=x1.device)
        wd = w.detach().to(dtype).contiguous()
        x1d = x1.detach().contiguous()
        if Z > 0:
            with torch.cuda.device(x1.device):
                stream = torch.cuda.current_stream(x1.device).cuda_stream
                code, es = _DTYPE_CODE[dtype], x1d.element_size()
                written = set()
                ranges = _row_ranges(Z, Cn, offsets)
                for p, count, da, dc in mod.fwd_groups:
                    cols = tuple(p.c_off + t * dc for t in range(count))
                    acc = 1 if any(c in written for c in cols) else 0
                    written.update(cols)
                    # out[z, k_seg] (+)= c * x1[z, i_seg] @ W_p[class(z)]; the K x N block is contraction-major as it lies
                    for lo, hi, offs in ranges:
                        _lib.check(
                            lib.cueq_gemm_grouped(code, code, 1, hi - lo, p.N, p.K, x1d.data_ptr() + (lo * x1d.stride(0) + p.a_off) * es,
                                                  x1d.stride(0), da, wd.data_ptr() + p.w_off * es, p.N, 0,
                                                  out.data_ptr() + (lo * out.stride(0) + p.c_off) * es, out.stride(0), dc,
                                                  count, offs.data_ptr(), Cn, 1, W, p.coeff, acc, stream),
                            "cueq_gemm_grouped",
                        )
        ctx.mod = mod
        ctx.save_for_backward(w, x1, offsets)
        return out

    @staticmethod
    def backward(ctx, g):
        # as for the shared-weight form: the two gradients are differentiable functions of their own
        mod = ctx.mod
        w, x1, offsets = ctx.saved_tensors
        gw = _IndexedDw.apply(mod, x1, g, w, offsets) if ctx.needs_input_grad[1] else None
        gx1 = _IndexedDx.apply(mod, g, w, offsets, x1) if ctx.needs_input_grad[2] else None
        return None, gw, gx1, None

    @staticmethod
    def grads(mod, w, x1, offsets, g, need_w, need_x1):
        dtype = x1.dtype
        Z, Cn, W = x1.shape[0], w.shape[0], w.shape[1]
        lib = _lib.load()
        g = g.detach().to(dtype).contiguous()
        wd = w.detach().to(dtype).contiguous()
        x1d = x1.detach().contiguous()
        gw = gx1 = None
        with torch.cuda.device(x1.device):
            stream = torch.cuda.current_stream(x1.device).cuda_stream
            code, es = _DTYPE_CODE[dtype], x1d.element_size()
            if need_x1:
                gx1 = (torch.empty_like if mod.dx1_covers_input else torch.zeros_like)(x1d)
                written = set()
                ranges = _row_ranges(Z, Cn, offsets)
                for p, count, dc, da in mod.dx1_groups if Z > 0 else []:
                    cols = tuple(p.a_off + t * da for t in range(count))
                    acc = 1 if any(c in written for c in cols) else 0
                    written.update(cols)
                    # dx1[z, i_seg] (+)= c * g[z, k_seg] @ W_p[class(z)]^T: the K x N block is "N' x K'" for this product
                    for lo, hi, offs in ranges:
                        _lib.check(
                            lib.cueq_gemm_grouped(code, code, 1, hi - lo, p.K, p.N, g.data_ptr() + (lo * g.stride(0) + p.c_off) * es, g.stride(0), dc,
                                                  wd.data_ptr() + p.w_off * es, p.N, 0, gx1.data_ptr() + (lo * gx1.stride(0) + p.a_off) * es,
                                                  gx1.stride(0), da, count, offs.data_ptr(), Cn, 0, W, p.coeff, acc, stream),
                            "cueq_gemm_grouped",
                        )
            if need_w:
                # dW_p[c] += coeff * sum over the rows z of class c of x1[z, i_seg]^T g[z, k_seg]: float32 accumulation
                gw32 = torch.zeros(Cn, W, dtype=torch.float32, device=x1.device)
                for p, count, da, dc in mod.fwd_groups if Z > 0 else []:
                    for t in range(count):
                        _lib.check(
                            lib.cueq_gemm_grouped(code, _lib.F32, 2, p.K, p.N, 0, x1d.data_ptr() + (p.a_off + t * da) * es, x1d.stride(0), 0,
                                                  g.data_ptr() + (p.c_off + t * dc) * es, g.stride(0), 0,
                                                  gw32.data_ptr() + p.w_off * 4, p.N, 0, 1, offsets.data_ptr(), Cn, 0, W, p.coeff, 1, stream),
                            "cueq_gemm_grouped",
                        )
                gw = gw32.to(w.dtype)
        return gw, gx1


class _IndexedDx(torch.autograd.Function):
    """``dx`` of the indexed Linear as a function of ``(g, w)``; ``x1`` gives the dtype of the result."""

    @staticmethod
    def forward(ctx, mod, g, w, offsets, x1):
        ctx.mod = mod
        ctx.save_for_backward(g, w, offsets)
        return _IndexedDenseFunction.grads(mod, w, x1, offsets, g, False, True)[1]

    @staticmethod
    def backward(ctx, c):
        g, w, offsets = ctx.saved_tensors
        dg = _IndexedDenseFunction.apply(ctx.mod, w, c, offsets).to(g.dtype) if ctx.needs_input_grad[1] else None
        dw = _IndexedDw.apply(ctx.mod, c, g, w, offsets) if ctx.needs_input_grad[2] else None
        return None, dg, dw, None, None


class _IndexedDw(torch.autograd.Function):
    """``dW`` (one row per class) of the indexed Linear as a function of ``(x1, g)``; ``w`` gives shape and dtype."""

    @staticmethod
    def forward(ctx, mod, x1, g, w, offsets):
        ctx.mod = mod
        ctx.save_for_backward(x1, g, offsets)
        return _IndexedDenseFunction.grads(mod, w, x1, offsets, g, True, False)[0]

    @staticmethod
    def backward(ctx, c):
        x1, g, offsets = ctx.saved_tensors
        dx = _IndexedDx.apply(ctx.mod, g, c, offsets, x1) if ctx.needs_input_grad[1] else None
        dg = _IndexedDenseFunction.apply(ctx.mod, c, x1, offsets).to(g.dtype) if ctx.needs_input_grad[2] else None
        return None, dx, dg, None, None


# ---------------------------------------------------------------------- traced execution (torch.compile / export)
# Forward and backward of the two shared-weight functions as opaque operators.  They call the static methods above with
# a plain object in place of the autograd context; the module travels as the text of its constructor's arguments, so
# that a graph saved by one process can be loaded by another (the module is then built again from that text).
_traced_modules: "OrderedDict[str, SegmentedPolynomialDense]" = OrderedDict()
_traced_lock = threading.Lock()
_FUNCTIONS = (_DenseFunction, _FcFunction)


class _PlainContext:
    def save_for_backward(self, *tensors):
        self.saved_tensors = tensors


def _module_by_key(key: str) -> "SegmentedPolynomialDense":
    with _traced_lock:
        mod = _traced_modules.get(key)
        if mod is not None:
            _traced_modules.move_to_end(key)
            return mod
    a = json.loads(key)
    return SegmentedPolynomialDense(cue.SegmentedPolynomial.unpack(a["polynomial"]), a["math_dtype"], a["output_dtype_map"], a["name"],
                                    a["method"], a["rows"], a["row_blocks"])  # (registers itself under the same text)


def _remember_traced(key: str, mod: "SegmentedPolynomialDense") -> None:
    with _traced_lock:
        _traced_modules[key] = mod
        while len(_traced_modules) > 256:
            _traced_modules.popitem(last=False)


@torch.library.custom_op("cuequivariance_amd::dense_fwd", mutates_args=(), device_types="cuda")
def _dense_fwd_op(mod_key: str, kind: int, w: torch.Tensor, x1: torch.Tensor, x2: Optional[torch.Tensor]) -> torch.Tensor:
    return _FUNCTIONS[kind].forward(_PlainContext(), _module_by_key(mod_key), w, x1, x2)


@_dense_fwd_op.register_fake
def _dense_fwd_fake(mod_key, kind, w, x1, x2):
    return x1.new_empty(x1.shape[0], _module_by_key(mod_key).out_size)


@torch.library.custom_op("cuequivariance_amd::dense_bwd", mutates_args=(), device_types="cuda")
def _dense_bwd_op(mod_key: str, kind: int, w: torch.Tensor, x1: torch.Tensor, x2: Optional[torch.Tensor], g: torch.Tensor,
                  need: List[bool]) -> List[torch.Tensor]:
    ctx = _PlainContext()
    ctx.mod, ctx.has_x2 = _module_by_key(mod_key), x2 is not None
    ctx.saved_tensors = (w, x1, x2 if (x2 is not None or kind == 1) else torch.empty(0))
    ctx.needs_input_grad = (False, *need)
    if kind == 0:
        grads = _DenseFunction._backward_impl(ctx, g, ctx.needs_input_grad)[1:4]
    else:
        grads = _FcFunction.grads(ctx.mod, w, x1, x2, g, *ctx.needs_input_grad[1:4])
    return [x1.new_empty(0) if (t is None or not n) else t.contiguous() for t, n in zip(grads, need)]


@_dense_bwd_op.register_fake
def _dense_bwd_fake(mod_key, kind, w, x1, x2, g, need):
    return [torch.empty_like(t) if (n and t is not None) else x1.new_empty(0) for t, n in zip((w, x1, x2), need)]


def _dense_setup_context(ctx, inputs, output):
    mod_key, kind, w, x1, x2 = inputs
    ctx.meta = (mod_key, kind, x2 is not None)
    ctx.save_for_backward(w, x1, *([x2] if x2 is not None else []))


def _dense_autograd(ctx, g):
    mod_key, kind, has_x2 = ctx.meta
    w, x1 = ctx.saved_tensors[:2]
    x2 = ctx.saved_tensors[2] if has_x2 else None
    need = [bool(n) for n in ctx.needs_input_grad[2:5]]
    got = _dense_bwd_op(mod_key, kind, w, x1, x2, g.contiguous(), need)
    gw, gx1, gx2 = [t if t.numel() > 0 else None for t in got]
    return None, None, gw, gx1, gx2


torch.library.register_autograd("cuequivariance_amd::dense_fwd", _dense_autograd, setup_context=_dense_setup_context)


def _apply_dense(kind: int, mod: "SegmentedPolynomialDense", w, x1, x2):
    if torch.compiler.is_compiling() or torch.jit.is_tracing() or type(x1) not in (torch.Tensor, torch.nn.Parameter):
        return _dense_fwd_op(mod.traced_key, kind, w, x1, x2)
    return _FUNCTIONS[kind].apply(mod, w, x1, x2)


class SegmentedPolynomialDense(nn.Module):
    """Dense (MFMA) executor for Linear / fully-connected polynomials with weights shared over the batch."""

    def __init__(self, polynomial: cue.SegmentedPolynomial, math_dtype=None, output_dtype_map: List[int] = None,
                 name: str = "segmented_polynomial", method: str = "fused_tp", rows: str = "ir_mul", row_blocks=None):
        super().__init__()
        self._polynomial_orig = polynomial
        self._rows_orig = rows
        self._row_blocks_orig = row_blocks
        self._output_dtype_map_orig = output_dtype_map
        self.name = name
        self.method = method
        if isinstance(math_dtype, str):
            math_dtype = getattr(torch, math_dtype)
        if math_dtype not in (None, torch.float32, torch.float64):
            raise ValueError("Fused TP only supports math_dtype==float32 or math_dtype==float64")
        self.math_dtype = math_dtype
        self.num_inputs, self.num_outputs = polynomial.num_inputs, polynomial.num_outputs
        self.input_sizes = [o.size for o in polynomial.inputs]
        self.out_size = polynomial.outputs[0].size
        self.paths, self.has_x2 = _analyse(polynomial)
        fwd, dx1 = {}, {}
        self.dw_groups: Dict[tuple, list] = {}
        for p in self.paths:
            fwd.setdefault((p.K, p.N), []).append((p.a_off, p.c_off, p.w_off, p.j, 0, p.coeff))
            dx1.setdefault((p.N, p.K), []).append((p.c_off, p.a_off, p.w_off, p.j, 1, p.coeff))
            self.dw_groups.setdefault((p.w_off, p.K, p.N), []).append(p)
        self.fwd_launches = _plan_gemm_launches(fwd)
        self.dx1_launches = _plan_gemm_launches(dx1)
        out_cols = sum(N for _, N, items, _ in self.fwd_launches for it in items if it[6] == 0)
        in_cols = sum(N for _, N, items, _ in self.dx1_launches for it in items if it[6] == 0)
        self.fwd_covers_output = out_cols == self.out_size
        self.dx1_covers_input = in_cols == self.input_sizes[1]
        self._tables: Dict[int, _DeviceTables] = {}
        # launches of the 128 x 128 tiled kernel (3-operand form only: no per-row scale there)
        self.fwd_groups = _batched_groups(self.paths, lambda p: p.a_off, lambda p: p.c_off)
        self.dx1_groups = _batched_groups(self.paths, lambda p: p.c_off, lambda p: p.a_off)
        self.weight_blocks = sorted({(p.w_off, p.K, p.N) for p in self.paths})
        self.fc_plan = _FcPlan(self.paths, self.input_sizes[2]) if self.has_x2 else None
        self._merged: dict = {}
        self._fused: dict = {}
        self._dw_shapes: dict = {}
        # rows="mul_ir": the irreps operands (input 1 and the output of the 3-operand form) keep the component index
        # contiguous inside every block; the kernels address them so - no transposition pass around the call.  Not part of
        # the reference's interface.  `mul_ir` is None when the blocks do not have the shape those kernels take.
        # 4-operand form: `row_blocks` = ([(mul, d)] of the first operand, [(mul, d)] of the output); the generated fused kernels
        # take such rows apart / put them together in registers, other executors of this module do not take them.
        self.mul_ir, self.fc_blocks = None, None
        if rows == "mul_ir" and not self.has_x2:
            self.mul_ir = _MulIrPlan.build(self)
            if self.mul_ir is None:
                raise NotImplementedError("fused_tp: rows='mul_ir' needs a Linear-like polynomial with blocks of 1, 3, 5 or 7 components "
                                          "and multiplicities 32, 64, 96 or 128")
        elif rows == "mul_ir":
            def starts(blocks, size):
                out, off = [], 0
                for mul, d in blocks:
                    out.append((off, int(mul), int(d)))
                    off += mul * d
                if off != size:
                    raise ValueError("fused_tp: row_blocks do not cover the operand")
                return out

            if row_blocks is None:
                raise NotImplementedError("fused_tp: rows='mul_ir' of a 4-operand contraction needs row_blocks")
            self.fc_blocks = (starts(row_blocks[0], self.input_sizes[1]), starts(row_blocks[1], self.out_size))
        self.rows_mul_ir = rows == "mul_ir"
        # the text under which a traced graph names this module: the arguments it was built from
        self.traced_key = json.dumps({
            "polynomial": polynomial.pack(), "math_dtype": None if math_dtype is None else str(math_dtype).split(".")[-1],
            "output_dtype_map": None if output_dtype_map is None else [int(i) for i in output_dtype_map], "name": name, "method": method,
            "rows": rows, "row_blocks": None if row_blocks is None else [[[int(m), int(d)] for m, d in blocks] for blocks in row_blocks]},
            separators=(",", ":"))
        _remember_traced(self.traced_key, self)

    def fused_unit(self, dtype, *row_tensors):
        """The kernels generated for this product (``codegen/fullyconnected.py``; compiled at first use), or ``None``:
        then the table-driven GEMMs run.  Rows are read and written in 16-byte pieces."""
        if dtype not in _MATRIX_CORE or not self.has_x2:
            return None
        if any(t.data_ptr() % 16 or (t.stride(0) * t.element_size()) % 16 or t.stride(1) != 1 for t in row_tensors):
            return None
        from .. import jit

        key = (dtype, jit.enabled())
        if key not in self._fused:
            blocks = self.fc_blocks or (None, None)
            self._fused[key] = jit.fully_connected_unit(self.paths, self.input_sizes[2], self.input_sizes[1], self.out_size,
                                                          _FC_ELEMENT[dtype], blocks[0], blocks[1])
        return self._fused[key]

    def mul_ir_ready(self, dtype) -> bool:
        """Whether rows in ``mul_ir`` can be taken as they lie for this dtype."""
        if not self.rows_mul_ir:
            return False
        if self.mul_ir is not None:
            return self.mul_ir.accepts(dtype)
        if dtype not in _MATRIX_CORE or not self.fc_plan.ok:
            return False
        from .. import jit

        key = (dtype, jit.enabled())
        if key not in self._fused:
            self._fused[key] = jit.fully_connected_unit(self.paths, self.input_sizes[2], self.input_sizes[1], self.out_size,
                                                          _FC_ELEMENT[dtype], *self.fc_blocks)
        return self._fused[key] is not None

    def tiled(self, dtype, A: torch.Tensor, Cout: torch.Tensor) -> bool:
        """The tiled kernel serves fp32 / bf16 contractions without a per-row scale."""
        return (not self.has_x2) and dtype in _MATRIX_CORE

    def transposed_weights(self, wd: torch.Tensor) -> torch.Tensor:
        """Every ``K x N`` weight block transposed in place of itself (same offsets) by ``cueq_transpose``."""
        lib = _lib.load()
        wt = torch.empty_like(wd)
        stream = torch.cuda.current_stream(wd.device).cuda_stream
        es = wd.element_size()
        for w_off, K, N in self.weight_blocks:
            _lib.check(lib.cueq_transpose(_DTYPE_CODE[wd.dtype], 1, K, N, wd.data_ptr() + w_off * es, wt.data_ptr() + w_off * es, stream),
                       "cueq_transpose")
        return wt

    def tables(self, device: torch.device) -> _DeviceTables:
        idx = device.index if device.index is not None else torch.cuda.current_device()
        t = self._tables.get(idx)
        if t is None:
            t = self._tables[idx] = _DeviceTables(self, torch.device("cuda", idx))
        return t

    def __reduce__(self):
        from .segmented_polynomial import SegmentedPolynomial

        return (SegmentedPolynomial, (self._polynomial_orig, self.method, self.math_dtype, self._output_dtype_map_orig, self.name,
                                      {"rows": self._rows_orig, "row_blocks": self._row_blocks_orig} if self._rows_orig != "ir_mul" else None))

    def _indexed(self, w: torch.Tensor, x1: torch.Tensor, index: torch.Tensor) -> torch.Tensor:
        """One weight row per class, rows of ``x1`` sorted by class (reference
        ``primitives/segmented_polynomial_indexed_linear.py:247-339``: sorted indices are required there too)."""
        if self.has_x2:
            raise NotImplementedError("indexed_linear: only the 3-operand (Linear) form is supported")
        if x1.device.type != "cuda":
            raise RuntimeError("indexed_linear runs on the GPU only; got tensors on " + str(x1.device))
        if x1.dtype not in _MATRIX_CORE:
            raise NotImplementedError(f"indexed_linear: float32, bfloat16 and float16 are implemented, got {x1.dtype}")
        if index.ndim != 1 or index.shape[0] != x1.shape[0]:
            raise ValueError("indexed_linear: the index must have one entry per batch row")
        Cn = w.shape[0]
        if index.numel() > 1:
            assert bool(torch.all(index[1:] - index[:-1] >= 0)), "Indexed_linear does not support non-sorted indices."
        counts = torch.bincount(index, minlength=Cn)
        if counts.shape[0] != Cn:
            raise ValueError("indexed_linear: an index is out of range of the weight rows")
        offsets = torch.zeros(Cn + 1, dtype=torch.int64, device=x1.device)
        offsets[1:] = torch.cumsum(counts, 0)
        return _IndexedDenseFunction.apply(self, w, x1, offsets)

    def forward(self, inputs: List[torch.Tensor], input_indices: Dict[int, torch.Tensor],
                output_shapes: Dict[int, torch.Tensor], output_indices: Dict[int, torch.Tensor]):
        for i, (x, size) in enumerate(zip(inputs, self.input_sizes)):
            if x.ndim != 2 or x.shape[-1] != size:
                raise ValueError(f"Input {i} has shape {tuple(x.shape)} but expected shape (rows, {size}).")
        w, x1 = inputs[0], inputs[1]
        if self.method == "indexed_linear" and set(input_indices) == {0} and not output_indices and not output_shapes:
            return [self._indexed(w, x1, input_indices[0])]
        if input_indices or output_indices or output_shapes:
            raise NotImplementedError(
                f"{self.method}: the dense executor takes weights shared over the batch, or (method='indexed_linear') "
                "weights indexed by a sorted class index; other indexed operands are not implemented")
        x2 = inputs[2] if self.has_x2 else None
        if x1.device.type != "cuda":
            raise RuntimeError("fused_tp runs on the GPU only; got tensors on " + str(x1.device))
        if w.shape[0] != 1:
            raise NotImplementedError("fused_tp: weights must be shared over the batch (one row)")
        if x1.dtype not in _DTYPE_CODE:
            raise ValueError(f"fused_tp: unsupported dtype {x1.dtype}")
        if self.rows_mul_ir and self.mul_ir is not None and not self.mul_ir.accepts(x1.dtype):
            raise NotImplementedError(f"fused_tp: rows='mul_ir' does not take {x1.dtype} with these multiplicities")
        if self.rows_mul_ir and self.fc_blocks is not None and not self.mul_ir_ready(x1.dtype):
            raise NotImplementedError("fused_tp: rows='mul_ir' of a fully connected product runs on the generated fused kernels only "
                                      "(float32 / bfloat16 / float16, compilation at first use switched on or the product prebuilt)")
        if self.math_dtype == torch.float32 and x1.dtype == torch.float64:
            raise ValueError("Fused TP does not support float32 math_dtype with float64 inputs.")
        if x2 is not None:
            if x2.dtype != x1.dtype:
                raise ValueError("fused_tp: both operands must have the same dtype")
            if x2.shape[0] == 1 and x1.shape[0] != 1:
                x2 = x2.expand(x1.shape[0], x2.shape[1])
            elif x1.shape[0] == 1 and x2.shape[0] != 1:
                x1 = x1.expand(x2.shape[0], x1.shape[1])
        if x2 is not None and x1.dtype == torch.float16 and not (self.fc_plan.ok and self.fused_unit(torch.float16, _aligned(x1.detach())) is not None):
            # half runs on the generated fused kernels only (the table-driven kernels behind them know float32 and bfloat16):
            # anything else is computed in float32 - every half is a float - and rounded once
            return [self.forward([w.float(), x1.float(), x2.float()], input_indices, output_shapes, output_indices)[0].to(torch.float16)]
        if x2 is not None and self.fc_plan.ok and x1.dtype in _MATRIX_CORE:
            return [_apply_dense(1, self, w, x1, x2)]
        return [_apply_dense(0, self, w, x1, x2)]
