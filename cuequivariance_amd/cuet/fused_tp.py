"""``method="fused_tp"``: the reference's dense 3- / 4-operand executor
(``cuequivariance_torch/cuequivariance_torch/primitives/segmented_polynomial_fused_tp.py:75-262``).

The reference accepts every polynomial whose operations have three or four operands and at least one path: its
dispatcher permutes the inputs and flattens modes until the operation fits one of eleven contraction forms
(``u__uw_w``, ``_v_vw_w``, ``u_v_uv_u``, ``u_v_uv_v``, ``u_u_uw_w``, ``u_v_uvw_w``, ``u_u_u``, ``u_v_uv``, ``u_uv_v``, ``u__u``,
``_v_v``; ``:114-160``), runs one fused operator per operation and adds the results per output buffer, with gathers of
indexed inputs and ``scatter_add_`` into indexed outputs (``:186-262``).

Here two executors stand behind the same interface:

* the matrix-core executor (``cuet/dense.py``) for what the high-level layers produce - one operation ``uv,iu,iv``
  (Linear) or ``uvw,iu,jv,kw`` with ``v = 1`` (fully connected product), weights shared over the batch, no index tensors;
* everything else - the other contraction forms, several operations, per-sample or indexed operands - on the
  uniform-1d kernels: every operation is flattened down to one channel mode (the last mode of its output, split to a
  common extent), which keeps gathers and scatters inside the kernels.  Correct for all the reference's forms, generated
  straight-line kernels at first use; these forms are element-wise / outer products without a matrix-core shape.
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
