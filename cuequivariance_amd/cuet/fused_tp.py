"""``method="fused_tp"``: the reference's dense 3- / 4-operand executor
(``cuequivariance_torch/cuequivariance_torch/primitives/segmented_polynomial_fused_tp.py:75-262``).

The reference accepts every polynomial whose operations have three or four operands and at least one path: its
dispatcher permutes the inputs and flattens modes until the operation fits one of eleven contraction forms
(``u__uw_w``, ``_v_vw_w``, ``u_v_uv_u``, ``u_v_uv_v``, ``u_u_uw_w``, ``u_v_uvw_w``, ``u_u_u``, ``u_v_uv``, ``u_uv_v``, ``u__u``,
``_v_v``; ``:114-160``), runs one fused operator per operation and adds the results per output buffer, with gathers of
indexed inputs and ``scatter_add_`` into indexed outputs (``:186-262``).

Here two executors stand behind the same interface:

* the matrix-core executor (``cuet/dense.py``) for what the high-level layers produce - one operation ``uv,iu,iv``
  (Linear) or ``uvw,iu,jv,kw`` with ``v = 1`` (fully connected product; also with that mode left out of the subscripts:
  ``u__uw_w``, ``_v_vw_w``), weights shared over the batch, no index tensors;
* the same executor behind an element-wise stage (``_MatrixWithElementwiseStage``) for the other forms with a matrix shape
  and shared weights: ``u_v_uvw_w`` with any ``v`` and ``u_u_uw_w`` (the products of the two row operands first, then their
  Linear map), ``u_v_uv_u`` and ``u_v_uv_v`` (the Linear map of one row operand first, then its product with the other);
* everything else - element-wise and outer products, several operations, per-sample or indexed operands - on the
  uniform-1d kernels: every operation is flattened down to one channel mode (the last mode of its output, split to a
  common extent), which keeps gathers and scatters inside the kernels.  Correct for all the reference's forms, generated
  straight-line kernels at first use.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch
import torch.nn as nn

from .. import cue

__all__ = ["SegmentedPolynomialFusedTP"]


class _FlattenedOperation(nn.Module):
    """One operation of a polynomial on the uniform-1d kernels: every mode but the last one of its output flattened
    away, that one split down to a common extent.  Built at first use."""

    def __init__(self, polynomial: cue.SegmentedPolynomial, math_dtype, output_dtype_map=None):
        super().__init__()
        self._polynomial, self._math_dtype, self._output_dtype_map = polynomial, math_dtype, output_dtype_map
        self.f = None

    def _build(self):
        from .segmented_polynomial import SegmentedPolynomial

        q = self._polynomial.flatten_coefficient_modes()
        stp = q.operations[0][1]
        ops = stp.subscripts.operands
        # the mode that stays must be the last subscript of every operand it appears in (the others are flattened from
        # the front): the output's last mode when that holds, else the admissible mode of largest extent (the output
        # then becomes scalar segments that contract it, e.g. u,v,uv,u keeps v), else none
        ok = [m for m in stp.subscripts.modes() if all(o.endswith(m) for o in ops if m in o)]
        keep = None
        if len(ops[-1]) and ops[-1][-1] in ok:
            keep = ops[-1][-1]
        elif ok:
            keep = max(ok, key=lambda m: max(stp.get_dims(m)))
        q = q.flatten_modes([m for m in stp.subscripts.modes() if m != keep])
        if keep is not None:
            extents = sorted(q.operations[0][1].get_dims(keep))
            if len(extents) > 1:
                q = q.split_mode(keep, math.gcd(*extents))
        return SegmentedPolynomial(q, method="uniform_1d", math_dtype=self._math_dtype, output_dtype_map=self._output_dtype_map)

    def forward(self, inputs, input_indices, output_shapes, output_indices):
        if self.f is None:
            self.f = self._build()
        return self.f(inputs, input_indices=input_indices, output_shapes=output_shapes, output_indices=output_indices)


class _MatrixWithElementwiseStage(nn.Module):
    """One 4-operand operation whose weights (the input with two or three modes) are shared over the batch, as a Linear map
    on the matrix-core executor and an element-wise stage; ``W`` stands for the weights, ``a`` and ``b`` for the two row
    operands in the order of the inputs, the names of the modes are free:

    * ``W[x y o], a[x], b[y] -> out[o]`` (``u_v_uvw_w``) and ``W[c o], a[c], b[c] -> out[o]`` (``u_u_uw_w``): the products
      ``P[z, (x, y)] = a[z, x] b[z, y]`` (or ``a[z, c] b[z, c]``) per distinct pair of segments, formed by broadcasting,
      then ``out = P W`` with ``W`` read as the ``(x y) x o`` matrix it is in memory.  The paths that add into one output
      segment become one path of the Linear map (their products side by side, their weight blocks stacked, each times its
      coefficient: a gather of the weight row), so no two paths write the same columns and the executor sends all paths of one
      contraction length out in one launch.  ``P`` has ``x y`` values per path and row: the rows are worked on in pieces that
      keep it under 4 GiB (``piece_bytes``); in training the products of all rows are kept for the weight gradient up to
      32 GiB (``keep_bytes``), beyond that every piece forms them again in the backward.
    * ``W[m0 m1], a, b -> out`` with one row operand carrying the contracted mode and the other the mode of the output
      (``u_v_uv_u``, ``u_v_uv_v``): ``T = g W`` (or ``g W^T``: the weights are gathered into that order first) per distinct
      (weight segment, segment of ``g``), then ``out += c e * T`` on the uniform-1d kernels.

    Everything between the stages is differentiable; 2-byte inputs stay 2-byte tensors on the first form (products and sums
    in float32, every tensor rounded once) and are computed in float32 on the others.  Raises
    ``NotImplementedError`` when the operation has none of these shapes."""

    def __init__(self, polynomial: cue.SegmentedPolynomial, math_dtype, name: str):
        super().__init__()
        import numpy as np

        from .dense import SegmentedPolynomialDense

        if len(polynomial.operations) != 1 or polynomial.num_inputs != 3 or polynomial.num_outputs != 1:
            raise NotImplementedError("one operation with three inputs and one output")
        ope, stp = polynomial.operations[0]
        if tuple(ope.buffers) != (0, 1, 2, 3) or stp.num_paths == 0:
            raise NotImplementedError("operands in buffer order")
        found = None
        for iw in range(3):
            sw = stp.subscripts.operands[iw]
            try:
                d = stp.flatten_modes([m for m in stp.subscripts.modes() if m not in sw])
            except ValueError:
                continue
            ia, ib = [i for i in range(3) if i != iw]
            W, a, b, o = (d.subscripts.operands[i] for i in (iw, ia, ib, 3))
            if len(W) == 3 and o == W[2] and {a, b} == {W[0], W[1]} and a != b:
                found = ("outer", d, iw, ia, ib, a == W[0])
            elif len(W) == 2 and a == b == W[0] and o == W[1]:
                found = ("same", d, iw, ia, ib, True)
            elif len(W) == 2 and len(a) == len(b) == 1 and {a, b} == {W[0], W[1]} and a != b and o in (a, b):
                g, e = (ia, ib) if o == b else (ib, ia)  # g carries the contracted mode, e the mode of the output
                found = ("after", d, iw, g, e, d.subscripts.operands[g] == W[0])
            if found:
                break
        if found is None:
            raise NotImplementedError(f"no matrix shape with shared weights in {stp.subscripts}")
        self.kind, d, self.iw, self.i1, self.i2, self.flag = found
        self.size = [o.size for o in d.operands]
        offs = [o.segment_offsets() for o in d.operands]
        lin = cue.SegmentedTensorProduct.from_subscripts("uv,u,v")
        paths = [(p.indices, float(p.coefficients)) for p in d.paths if float(p.coefficients) != 0.0]
        if not paths:
            raise NotImplementedError("no path with a coefficient")
        self.w_gather, self.w_scale = None, None
        if self.kind in ("outer", "same"):
            # The paths that add into one output segment are one product: out[:, c] = [P_1 | P_2 | ...] [c_1 W_1; c_2 W_2; ...]
            # (their products side by side, their weight blocks stacked, each times its coefficient), so the Linear map has one
            # path per output segment, no two of them write the same columns, and all of one contraction length go out in one
            # table-driven launch.  Products are formed together per shape (extent of a, extent of b): with mixed shapes an
            # output segment has one such path per shape.
            by_shape = {}
            for idx, c in paths:
                na, nb = d.operands[self.i1][idx[self.i1]][0], d.operands[self.i2][idx[self.i2]][0]
                by_shape.setdefault((na, nb), {}).setdefault(idx[3], []).append((idx, c))
            for seg in d.operands[3]:
                lin.add_segment(2, tuple(seg))
            self.groups, gather, scale = [], [], []
            self.parts, cursor = [], 0  # (kind "outer": every product as (offset in a, in b, in P, extent of a, of b), in the order of P)
            for (na, nb), by_out in sorted(by_shape.items()):
                k = na * nb if self.kind == "outer" else na
                rows_a, rows_b = [], []
                for out_seg, members in sorted(by_out.items()):
                    n = d.operands[3][out_seg][0]
                    sw = lin.add_segment(0, (k * len(members), n))
                    sp = lin.add_segment(1, (k * len(members),))
                    lin.add_path(sw, sp, out_seg, c=1.0)
                    for idx, c in members:
                        rows_a.append([offs[self.i1][idx[self.i1]] + t for t in range(na)])
                        rows_b.append([offs[self.i2][idx[self.i2]] + t for t in range(nb)])
                        self.parts.append((offs[self.i1][idx[self.i1]], offs[self.i2][idx[self.i2]], cursor, na, nb))
                        cursor += k
                        gather.append(offs[self.iw][idx[self.iw]] + np.arange(k * n))
                        scale.append(np.full(k * n, c))
                self.groups.append((torch.tensor(rows_a), torch.tensor(rows_b)))
            self.w_gather = torch.from_numpy(np.concatenate(gather))
            self.w_scale = torch.from_numpy(np.concatenate(scale))
            self.after = None
        else:
            transposed = not self.flag  # the weights lie (output mode, contracted mode): gathered into the other order
            if transposed:
                gather = np.arange(self.size[self.iw])
                for seg, off in zip(d.operands[self.iw], offs[self.iw]):
                    gather[off:off + seg[0] * seg[1]] = off + np.arange(seg[0] * seg[1]).reshape(seg[0], seg[1]).T.reshape(-1)
                self.w_gather = torch.from_numpy(gather)
            for seg in d.operands[self.iw]:
                lin.add_segment(0, (seg[1], seg[0]) if transposed else tuple(seg))
            for seg in d.operands[self.i1]:
                lin.add_segment(1, tuple(seg))
            uses = sorted({(idx[self.iw], idx[self.i1]) for idx, _ in paths})
            el = cue.SegmentedTensorProduct.from_subscripts("u,u,u")
            for seg in d.operands[self.i2]:
                el.add_segment(0, tuple(seg))
            for t, (pw, pg) in enumerate(uses):
                n = lin.operands[0][pw][1]
                lin.add_segment(2, (n,))
                el.add_segment(1, (n,))
                lin.add_path(pw, pg, t, c=1.0)
            for seg in d.operands[3]:
                el.add_segment(2, tuple(seg))
            for idx, c in paths:
                el.add_path(idx[self.i2], uses.index((idx[self.iw], idx[self.i1])), idx[3], c=c)
            self.groups = []
            self.after = _FlattenedOperation(
                cue.SegmentedPolynomial([el.operands[0], el.operands[1]], [el.operands[2]], [(cue.Operation([0, 1, 2]), el)]), math_dtype)
        self.p_size = lin.operands[1].size
        # what the flattened operation would have to walk per row: one scalar path per contracted index of every path
        self.scalar_paths = sum(lin.operands[0][p.indices[0]][0] for p in lin.paths)
        self.linear = SegmentedPolynomialDense(
            cue.SegmentedPolynomial([lin.operands[0], lin.operands[1]], [lin.operands[2]], [(cue.Operation([0, 1, 2]), lin)]),
            math_dtype, None, name)
        self._on_device: dict = {}
        # rows are worked on in pieces whose products take at most this many bytes (large pieces fill the chip better: the
        # Linear map has few, long contractions)
        self.piece_bytes = 4 << 30
        # products of all rows beyond this many bytes are not kept for the backward but formed again there
        self.keep_bytes = 32 << 30

    def _tables(self, device):
        t = self._on_device.get(device)
        if t is None:
            t = self._on_device[device] = ([(ga.to(device), gb.to(device)) for ga, gb in self.groups],
                                           None if self.w_gather is None else self.w_gather.to(device),
                                           None if self.w_scale is None else self.w_scale.to(device))
        return t

    def outer_tables(self, device):
        """Device tables of ``cueq_outer_rows`` / ``cueq_outer_rows_contract`` for the products of this stage: the parts, and
        per row operand the parts that read each of its segments (in the order of P: the order the sums take)."""
        key = ("outer", device)
        t = self._on_device.get(key)
        if t is None:
            parts = torch.tensor(self.parts, dtype=torch.int32)
            lists = []
            for col in (0, 1):  # segments of a, of b
                by_seg = {}
                for q, part in enumerate(self.parts):
                    by_seg.setdefault(part[col], []).append(q)
                start, members = [0], []
                for _, qs in sorted(by_seg.items()):
                    members += qs
                    start.append(len(members))
                lists.append((torch.tensor(start, dtype=torch.int32).to(device), torch.tensor(members, dtype=torch.int32).to(device),
                              len(start) - 1, max(self.parts[qs[0]][3 + col] for qs in by_seg.values())))
            vec = 8 if all(v % 8 == 0 for part in self.parts for v in part) else 4 if all(v % 4 == 0 for part in self.parts for v in part) else 0
            t = self._on_device[key] = (parts.to(device), len(self.parts), max(na * nb for _, _, _, na, nb in self.parts), lists, vec)
        return t

    def forward(self, inputs: List[torch.Tensor]) -> torch.Tensor:
        traced = torch.compiler.is_compiling() or torch.jit.is_tracing()
        if inputs[0].dtype in (torch.bfloat16, torch.float16) and (self.kind != "outer" or traced):
            # (2-byte inputs stay what they are on the product kernels and the matrix cores only: products and sums in float32,
            # every tensor rounded once; the stages in torch code are computed in float32 throughout)
            inputs = [t.float() for t in inputs]
        w, x1, x2 = inputs[self.iw], inputs[self.i1], inputs[self.i2]
        groups, w_gather, w_scale = self._tables(w.device)
        Z = max(x1.shape[0], x2.shape[0])
        if self.kind == "after":
            if w_gather is not None:
                w = w[:, w_gather]
            t = self.linear([w, x1.contiguous()], {}, {}, {})[0]
            return self.after([x2, t], {}, {}, {})[0]
        if Z == 0:  # (no rows: nothing to launch; the result still hangs on the inputs)
            return x1.new_zeros((0, self.size[3])) + 0 * (x1.sum() + x2.sum() + w.sum())
        # the weight blocks of every path, stacked per output segment, times the coefficients (2-byte weights: rounded once)
        w = (w.float()[:, w_gather] * w_scale.float()).to(w.dtype) if w.dtype in (torch.bfloat16, torch.float16) else w[:, w_gather] * w_scale.to(w.dtype)
        step = max(1, self.piece_bytes // max(1, self.p_size * w.element_size()))

        def piece(a, b, w):
            rows = max(a.shape[0], b.shape[0])
            if self.kind == "outer" and not traced:
                # (the kernels of csrc/outer_rows.hip; a traced graph keeps the torch code below)
                return self.linear([w, _OuterRows.apply(self, a.expand(rows, -1), b.expand(rows, -1))], {}, {}, {})[0]
            parts = []
            for ga, gb in groups:
                if self.kind == "same":
                    prod = a[:, ga] * b[:, gb]
                elif self.flag:  # the mode of a comes first in the weights
                    prod = a[:, ga][:, :, :, None] * b[:, gb][:, :, None, :]
                else:
                    prod = b[:, gb][:, :, :, None] * a[:, ga][:, :, None, :]
                parts.append(prod.expand(rows, *prod.shape[1:]).reshape(rows, -1))
            return self.linear([w, parts[0] if len(parts) == 1 else torch.cat(parts, 1)], {}, {}, {})[0]

        # The weight gradient needs the products again: autograd keeps them, all pieces of them, until the backward.  Beyond
        # `keep_bytes` they are formed a second time in the backward instead, piece by piece (one more product kernel per piece).
        again = (not traced and torch.is_grad_enabled() and Z * self.p_size * w.element_size() > self.keep_bytes
                 and any(t.requires_grad for t in (x1, x2, w)))
        outs = []
        for z0 in range(0, Z, step):
            a = x1 if x1.shape[0] == 1 else x1[z0:z0 + step]
            b = x2 if x2.shape[0] == 1 else x2[z0:z0 + step]
            if x1.shape[0] == 1 and x2.shape[0] == 1:
                b = b.expand(min(step, Z - z0), -1)
            if again:
                from torch.utils.checkpoint import checkpoint

                outs.append(checkpoint(piece, a, b, w, use_reentrant=False))
            else:
                outs.append(piece(a, b, w))
        return outs[0] if len(outs) == 1 else torch.cat(outs, 0)


def _code(dtype):
    from .. import _lib

    return {torch.float32: _lib.F32, torch.float64: _lib.F64, torch.bfloat16: _lib.BF16, torch.float16: _lib.F16}[dtype]


def _outer_launch(st: "_MatrixWithElementwiseStage", a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    from .. import _lib

    a, b = a.contiguous(), b.contiguous()
    rows = a.shape[0]
    parts, nparts, max_part, _, vec = st.outer_tables(a.device)
    out = torch.empty(rows, st.p_size, dtype=a.dtype, device=a.device)
    with torch.cuda.device(a.device):
        _lib.check(_lib.load().cueq_outer_rows(
            _code(a.dtype), rows, a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0), out.data_ptr(),
            out.stride(0), parts.data_ptr(), nparts, max_part, 1 if st.flag else 0, vec,
            torch.cuda.current_stream(a.device).cuda_stream), "cueq_outer_rows")
    return out


def _contract_launch(st: "_MatrixWithElementwiseStage", which: int, q: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    from .. import _lib

    q, x = q.contiguous(), x.contiguous()
    rows = q.shape[0]
    parts, _, _, lists, vec = st.outer_tables(q.device)
    start, members, nsegs, max_extent = lists[which]
    out = torch.zeros(rows, st.size[st.i1 if which == 0 else st.i2], dtype=q.dtype, device=q.device)
    with torch.cuda.device(q.device):
        _lib.check(_lib.load().cueq_outer_rows_contract(
            _code(q.dtype), which, rows, q.data_ptr(), q.stride(0), x.data_ptr(), x.stride(0),
            out.data_ptr(), out.stride(0), parts.data_ptr(), start.data_ptr(), members.data_ptr(), nsegs, max_extent,
            1 if st.flag else 0, vec, torch.cuda.current_stream(q.device).cuda_stream), "cueq_outer_rows_contract")
    return out


class _OuterRows(torch.autograd.Function):
    """``P = a (x) b`` per part (``cueq_outer_rows``).  Its gradients are the two contractions of ``_ContractRows``, whose
    gradients are this product and the other contraction: derivatives of any order stay on the three kernels."""

    @staticmethod
    def forward(ctx, st, a, b):
        ctx.st = st
        ctx.save_for_backward(a, b)
        return _outer_launch(st, a.detach(), b.detach())

    @staticmethod
    def backward(ctx, g):
        a, b = ctx.saved_tensors
        return (None, _ContractRows.apply(ctx.st, 0, g, b) if ctx.needs_input_grad[1] else None,
                _ContractRows.apply(ctx.st, 1, g, a) if ctx.needs_input_grad[2] else None)


class _ContractRows(torch.autograd.Function):
    """``which = 0``: ``out[z, u] = sum_p sum_v q[z, p, u, v] x[z, v]`` (``x`` in the place of ``b``); ``which = 1``: the sum over
    ``u`` with ``x`` in the place of ``a`` (``cueq_outer_rows_contract``)."""

    @staticmethod
    def forward(ctx, st, which, q, x):
        ctx.st, ctx.which = st, which
        ctx.save_for_backward(q, x)
        return _contract_launch(st, which, q.detach(), x.detach())

    @staticmethod
    def backward(ctx, c):
        q, x = ctx.saved_tensors
        st, which = ctx.st, ctx.which
        gq = gx = None
        if ctx.needs_input_grad[2]:
            gq = _OuterRows.apply(st, c, x) if which == 0 else _OuterRows.apply(st, x, c)
        if ctx.needs_input_grad[3]:
            gx = _ContractRows.apply(st, 1 - which, q, c)
        return None, None, gq, gx


def _permute_inputs(polynomial: cue.SegmentedPolynomial, perm) -> cue.SegmentedPolynomial:
    """The same polynomial with input ``perm[k]`` of the original in position ``k``."""
    nin = polynomial.num_inputs
    new_id = {old: new for new, old in enumerate(perm)}
    ops = [(cue.Operation([new_id[b] if b < nin else b for b in ope.buffers]), stp) for ope, stp in polynomial.operations]
    return cue.SegmentedPolynomial([polynomial.inputs[i] for i in perm], polynomial.outputs, ops)


class SegmentedPolynomialFusedTP(nn.Module):
    def __init__(self, polynomial: cue.SegmentedPolynomial, math_dtype=None, output_dtype_map: Optional[List[int]] = None,
                 name: str = "segmented_polynomial", rows: str = "ir_mul", row_blocks=None):
        super().__init__()
        from .dense import SegmentedPolynomialDense

        self._rows_orig, self._row_blocks_orig = rows, row_blocks

        self._polynomial_orig = polynomial
        self._output_dtype_map_orig = output_dtype_map
        self.num_inputs, self.num_outputs = polynomial.num_inputs, polynomial.num_outputs
        self.input_sizes = [o.size for o in polynomial.inputs]
        self.out_size = [o.size for o in polynomial.outputs]
        self.name = name
        # (the reference turns a missing math_dtype into float32 with a warning and then refuses float64 inputs; here a
        # missing math_dtype follows the inputs: float64 inputs are computed in float64, everything else in float32)
        if isinstance(math_dtype, str):
            try:
                math_dtype = getattr(torch, math_dtype)
            except AttributeError:
                raise ValueError(f"Math_dtype {math_dtype} is not accepted for method `fused_tp`.")
        if math_dtype not in (None, torch.float32, torch.float64):
            raise ValueError("Fused TP only supports math_dtype==float32 or math_dtype==float64")
        self.math_dtype = math_dtype
        default_map = [0 if polynomial.num_inputs >= 1 else -1] * polynomial.num_outputs
        self.dtypes = list(range(self.num_inputs)) + (default_map if output_dtype_map is None else list(output_dtype_map))
        for _, d in polynomial.operations:
            if d.num_paths == 0:
                raise NotImplementedError("Fused TP does not support empty paths.")
            if d.num_operands not in (3, 4):
                raise NotImplementedError(f"Fused TP only supports 3 or 4 operands. Got {d.subscripts}.")
        # the matrix-core executor wants the weights first (uv,iu,iv / uvw,iu,jv,kw): like the reference's dispatcher, try
        # the orders of the inputs
        self.dense, self.dense_perm = None, None
        if len(polynomial.operations) == 1 and polynomial.num_outputs == 1 and polynomial.num_inputs in (2, 3):
            import itertools

            for perm in itertools.permutations(range(polynomial.num_inputs)):
                try:
                    if rows == "mul_ir" and perm != tuple(range(polynomial.num_inputs)):
                        continue  # (row_blocks name the operands in the given order)
                    self.dense = SegmentedPolynomialDense(_permute_inputs(polynomial, perm), math_dtype, output_dtype_map, name, rows=rows,
                                                          row_blocks=row_blocks)
                    self.dense_perm = perm
                    break
                except NotImplementedError:
                    continue
        # the other forms with a matrix shape: a Linear map on the same executor and an element-wise stage, taken when the
        # flattened operation would have `stages_from` scalar paths or more (small multiplicities are one cheap launch of a
        # generated uniform-1d kernel; beyond a few thousand paths that kernel takes minutes to compile and the matrix
        # cores are far ahead)
        self.stages_from = 2048
        self.composed = None
        if self.dense is None and rows != "mul_ir":
            try:
                self.composed = _MatrixWithElementwiseStage(polynomial, math_dtype, name)
            except NotImplementedError:
                self.composed = None
        if rows == "mul_ir" and self.dense is None:
            raise NotImplementedError("fused_tp: rows='mul_ir' is served by the matrix-core executor only")
        # one flattened executor per operation: (module, input buffers it reads, output it adds to)
        self.ops = nn.ModuleList()
        self.op_inputs, self.op_output = [], []
        for ope, stp in polynomial.operations:
            ins = sorted(set(ope.input_buffers(self.num_inputs)))
            b_out = ope.output_buffer(self.num_inputs)
            local = [ins.index(b) if b < self.num_inputs else len(ins) for b in ope.buffers]
            sub = cue.SegmentedPolynomial([polynomial.inputs[b] for b in ins], [polynomial.outputs[b_out - self.num_inputs]],
                                          [(cue.Operation(local), stp)])
            # the operation's result in the type the polynomial's output is to have (the reference sums in that type): the
            # input it inherits from when the operation reads it, else the arithmetic type - rounded once, after the sum
            src = self.dtypes[b_out]
            self.ops.append(_FlattenedOperation(sub, math_dtype, [ins.index(src) if src in ins else -1]))
            self.op_inputs.append(ins)
            self.op_output.append(b_out - self.num_inputs)

    def __reduce__(self):
        from .segmented_polynomial import SegmentedPolynomial

        return (SegmentedPolynomial, (self._polynomial_orig, "fused_tp", self.math_dtype, self._output_dtype_map_orig, self.name,
                                      {"rows": self._rows_orig, "row_blocks": self._row_blocks_orig} if self._rows_orig != "ir_mul" else None))

    def forward(self, inputs: List[torch.Tensor], input_indices: Dict[int, torch.Tensor],
                output_shapes: Dict[int, torch.Tensor], output_indices: Dict[int, torch.Tensor]):
        for i, (x, size) in enumerate(zip(inputs, self.input_sizes)):
            if x.ndim == 0:
                raise ValueError(f"Input {i} has no dimensions")
            if x.shape[-1] != size:
                raise ValueError(f"Input {i} has shape {x.shape} but expected shape {size}.")
        if self.math_dtype == torch.float32 and any(t.dtype == torch.float64 for t in inputs):
            raise ValueError("Fused TP does not support float32 math_dtype with float64 inputs.")
        for k in output_indices:
            assert k in output_shapes, "output shapes must be provided for output indices"
        if (self.dense is not None and not input_indices and not output_indices and not output_shapes
                and inputs[self.dense_perm[0]].shape[0] == 1 and inputs[0].dtype in (torch.float32, torch.float64, torch.bfloat16, torch.float16)
                and all(t.dtype == inputs[0].dtype for t in inputs)):
            return self.dense([inputs[i] for i in self.dense_perm], input_indices, output_shapes, output_indices)
        if (self.composed is not None and self.composed.scalar_paths >= self.stages_from and not input_indices and not output_indices and not output_shapes and inputs[0].is_cuda
                and inputs[self.composed.iw].shape[0] == 1 and inputs[0].dtype in (torch.float32, torch.float64, torch.bfloat16, torch.float16)
                and all(t.dtype == inputs[0].dtype for t in inputs)
                and len({t.shape[0] for i, t in enumerate(inputs) if i != self.composed.iw} - {1}) <= 1):
            out = self.composed(inputs)
            src = self.dtypes[self.num_inputs]
            dtype = (self.math_dtype or torch.float32) if src < 0 else inputs[src].dtype
            return [out if out.dtype == dtype else out.to(dtype)]
        if self._rows_orig == "mul_ir":
            raise NotImplementedError("fused_tp: rows='mul_ir' takes shared weights, no index tensors and one dtype for all inputs")
        device = inputs[0].device
        outs: List[Optional[torch.Tensor]] = [None] * self.num_outputs
        for f, ins, o in zip(self.ops, self.op_inputs, self.op_output):
            r = f([inputs[b] for b in ins],
                  {ins.index(b): v for b, v in input_indices.items() if b in ins},
                  {0: output_shapes[o]} if o in output_shapes else {},
                  {0: output_indices[o]} if o in output_indices else {})[0]
            if outs[o] is None:
                outs[o] = r
            elif outs[o].shape[0] == r.shape[0] or r.shape[0] == 1:
                outs[o] = outs[o] + r
            elif outs[o].shape[0] == 1:
                outs[o] = r + outs[o]
            else:
                raise ValueError(f"Input/output batch size mismatch {outs[o].shape} vs {r.shape}.")
        batch = max([1] + [t.shape[0] for i, t in enumerate(inputs) if i not in input_indices] + [v.shape[0] for v in input_indices.values()])
        result = []
        for o in range(self.num_outputs):
            src = self.dtypes[self.num_inputs + o]
            dtype = (self.math_dtype or torch.float32) if src < 0 else inputs[src].dtype
            if outs[o] is None:  # no operation writes this output
                rows = output_shapes[o].shape[0] if o in output_shapes else batch
                result.append(torch.zeros(rows, self.out_size[o], dtype=dtype, device=device))
            else:
                result.append(outs[o] if outs[o].dtype == dtype else outs[o].to(dtype))
        return result
