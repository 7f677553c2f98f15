"""TEST INFRASTRUCTURE ONLY - CPU restatement of the reference's executor for segmented polynomials.

Nothing under ``cuequivariance_amd/`` may import this module.  It exists so that tests, the smoke
check and the CPU-baseline leg of the benchmark can compare the HIP kernels with the reference's
algorithm on the same inputs.

What it restates (paths relative to the reference checkout):

* ``cuequivariance_torch/cuequivariance_torch/primitives/segmented_polynomial_naive.py:61-160``
  ``_tensor_product_fx``: per path, slice the operand segments, reshape, cast to ``math_dtype``,
  ``einsum(coeff, seg_0, seg_1, ...)``, cast back to the dtype of the first input; paths are summed
  per output segment in path order; segments are concatenated.
* same file ``:360-435`` ``SegmentedPolynomialNaive.forward``: gather indexed inputs first
  (``x[idx]``), run every operation, then ``zeros(rows, size).scatter_add_(0, idx, out)`` for indexed
  outputs, ``sum(0)`` when the output has one row, broadcast when the result has one row.
* ``cuequivariance/cuequivariance/segmented_polynomials/evaluate.py:25-139`` (numpy twin, see
  :func:`numpy_last_operand`).

The polynomial is passed as a plain *spec* (see :func:`spec_from_polynomial`) so that this file does
not depend on the descriptor classes of the package under test.

Pinned by ``tests/test_oracle.py``: brute-force loops on tiny descriptors, matmul identities
(the reference's ``evaluate_test.py:20-104``), gather/scatter identity
(``cuequivariance_torch/tests/operations/channel_wise_test.py:231-305``), and a closed-form
channel-wise product written out in that test file.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch


def spec_from_polynomial(poly) -> dict:
    """Plain-data description of a segmented polynomial (duck-typed: any object with the same attributes)."""
    ops = []
    for ope, stp in poly.operations:
        ops.append(
            dict(
                buffers=list(ope.buffers),
                operand_subscripts=list(stp.subscripts.operands),
                coefficient_subscripts=str(stp.coefficient_subscripts),
                segments=[[tuple(s) for s in o.segments] for o in stp.operands],
                path_indices=[tuple(p.indices) for p in stp.paths],
                path_coefficients=[np.array(p.coefficients, dtype=np.float64) for p in stp.paths],
            )
        )
    return dict(
        num_inputs=poly.num_inputs,
        num_outputs=poly.num_outputs,
        sizes=[o.size for o in poly.operands],
        operations=ops,
    )


def _offsets(segments) -> List[int]:
    out, off = [], 0
    for s in segments:
        out.append(off)
        off += math.prod(s)
    return out


def _tensor_product(op: dict, out_pos: int, inputs: List[torch.Tensor], math_dtype: Optional[torch.dtype],
                    first_dtype: torch.dtype) -> torch.Tensor:
    """One operation: inputs ``(Z | 1, operand_size)`` in operand order (output slot skipped) -> ``(Z, out_size)``."""
    nops = len(op["buffers"])
    in_pos = [k for k in range(nops) if k != out_pos]
    ss = op["operand_subscripts"]
    formula = ",".join([op["coefficient_subscripts"]] + ["Z" + ss[k] for k in in_pos]) + "->Z" + ss[out_pos]
    offs = [_offsets(segs) for segs in op["segments"]]
    out_segments = op["segments"][out_pos]
    if not in_pos:
        # an operation without inputs is a constant row (segmented_polynomial_naive.py:184-240), broadcast by the caller
        row = torch.zeros(sum(math.prod(sh) for sh in out_segments), dtype=math_dtype or torch.float64)
        for idx, coeff in zip(op["path_indices"], op["path_coefficients"]):
            shape = out_segments[idx[out_pos]]
            o = offs[out_pos][idx[out_pos]]
            row[o: o + math.prod(shape)] += torch.tensor(coeff, dtype=row.dtype).reshape(-1)
        return row.to(first_dtype).reshape(1, -1)
    per_segment: List[List[torch.Tensor]] = [[] for _ in out_segments]
    for idx, coeff in zip(op["path_indices"], op["path_coefficients"]):
        if not np.any(coeff != 0):
            continue  # remove_zero_paths
        segs = []
        for x, k in zip(inputs, in_pos):
            shape = op["segments"][k][idx[k]]
            o = offs[k][idx[k]]
            seg = x[..., o: o + math.prod(shape)].reshape(x.shape[:-1] + tuple(shape))
            segs.append(seg.to(math_dtype) if math_dtype is not None else seg)
        if math_dtype is not None:
            c = torch.tensor(coeff, dtype=math_dtype)
        else:
            c = torch.tensor(coeff, dtype=torch.float64).to(first_dtype)
        r = torch.einsum(formula, c, *segs)
        if math_dtype is not None:
            r = r.to(first_dtype)
        per_segment[idx[out_pos]].append(r.reshape(r.shape[0], -1))
    batch = max([x.shape[0] for x in inputs] + [1])
    cols = []
    for seg_shape, parts in zip(out_segments, per_segment):
        if not parts:
            cols.append(torch.zeros((batch, math.prod(seg_shape)), dtype=first_dtype))
            continue
        acc = parts[0]
        for p in parts[1:]:
            acc = torch.add(acc, p)
        cols.append(acc.expand(batch, acc.shape[1]) if acc.shape[0] != batch else acc)
    return torch.cat(cols, dim=-1)


def naive_segmented_polynomial(
    spec: dict,
    inputs: Sequence[torch.Tensor],
    input_indices: Optional[Dict[int, torch.Tensor]] = None,
    output_shapes: Optional[Dict[int, int]] = None,
    output_indices: Optional[Dict[int, torch.Tensor]] = None,
    math_dtype: Optional[torch.dtype] = None,
    output_dtype_map: Optional[Sequence[int]] = None,
) -> List[torch.Tensor]:
    """Evaluate on CPU tensors.  ``output_shapes[k]`` is the row count of output ``k``.  Differentiable (autograd)."""
    input_indices = input_indices or {}
    output_shapes = output_shapes or {}
    output_indices = output_indices or {}
    nin, nout = spec["num_inputs"], spec["num_outputs"]
    inputs = list(inputs)
    assert len(inputs) == nin
    for i, x in enumerate(inputs):
        if x.shape[-1] != spec["sizes"][i]:
            raise ValueError(f"Input {i} has shape {tuple(x.shape)} but expected size {spec['sizes'][i]}.")
    for k, idx in input_indices.items():
        inputs[k] = inputs[k][idx.long()]
    batch = 1
    for x in inputs:
        if x.shape[0] != 1:
            assert batch in (1, x.shape[0])
            batch = x.shape[0]
    first_dtype = inputs[0].dtype
    dmap = list(output_dtype_map) if output_dtype_map is not None else [0 if nin >= 1 else -1] * nout
    out_rows = [output_shapes.get(o, batch) for o in range(nout)]
    outs: List[Optional[torch.Tensor]] = [None] * nout
    for op in spec["operations"]:
        out_pos = [k for k, b in enumerate(op["buffers"]) if b >= nin]
        assert len(out_pos) == 1
        out_pos = out_pos[0]
        o = op["buffers"][out_pos] - nin
        res = _tensor_product(op, out_pos, [inputs[b] for k, b in enumerate(op["buffers"]) if k != out_pos],
                              math_dtype, first_dtype)
        size = spec["sizes"][nin + o]
        if o in output_indices:
            idx = output_indices[o].long()
            if res.shape[0] == 1 and idx.shape[0] > 1:
                res = res.expand(idx.shape[0], res.shape[1])
            odt = inputs[dmap[o]].dtype if dmap[o] >= 0 else (math_dtype or first_dtype)
            tmp = torch.zeros((out_rows[o], size), dtype=odt).scatter_add(0, idx.unsqueeze(-1).expand_as(res), res.to(odt))
        elif out_rows[o] == res.shape[0]:
            tmp = res
        elif out_rows[o] == 1:
            tmp = res.sum(dim=0, keepdim=True)
        elif res.shape[0] == 1:
            tmp = res.expand(out_rows[o], size).clone()
        else:
            raise ValueError(f"Input/output batch size mismatch {out_rows[o]} vs {res.shape}.")
        outs[o] = tmp if outs[o] is None else outs[o] + tmp
    for o in range(nout):
        if outs[o] is None:
            outs[o] = torch.zeros((out_rows[o], spec["sizes"][nin + o]), dtype=first_dtype)
    return outs


def numpy_last_operand(op: dict, *inputs: np.ndarray) -> np.ndarray:
    """numpy evaluation of one operation whose output is the last operand (``evaluate.py:89-139``)."""
    ss = op["operand_subscripts"]
    formula = ",".join([op["coefficient_subscripts"]] + ["..." + s for s in ss[:-1]]) + "->..." + ss[-1]
    offs = [_offsets(segs) for segs in op["segments"]]
    batch = np.broadcast_shapes(*[x.shape[:-1] for x in inputs])
    out = np.zeros(batch + (sum(math.prod(s) for s in op["segments"][-1]),), dtype=np.result_type(*inputs))
    for idx, coeff in zip(op["path_indices"], op["path_coefficients"]):
        segs = []
        for k, x in enumerate(inputs):
            shape = op["segments"][k][idx[k]]
            o = offs[k][idx[k]]
            segs.append(x[..., o: o + math.prod(shape)].reshape(x.shape[:-1] + tuple(shape)))
        r = np.einsum(formula, coeff, *segs)
        shape = op["segments"][-1][idx[-1]]
        o = offs[-1][idx[-1]]
        out[..., o: o + math.prod(shape)] += r.reshape(batch + (-1,))
    return out
