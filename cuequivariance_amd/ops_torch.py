"""The operator seam of the reference's torch frontend, served by this engine.

``cuequivariance_torch`` reaches its closed kernels through a package named ``cuequivariance_ops_torch``:

* ``cuequivariance_ops_torch.uniform_1d.BATCH_DIM_*`` and ``torch.ops.cuequivariance.uniform_1d(...)``
  (``cuequivariance_torch/primitives/segmented_polynomial_uniform_1d.py:25-30, 55-77``),
* ``segmented_transpose(x, info, contiguous)`` (``primitives/transpose.py:172-183``, ``info`` rows
  ``[offset, u, v, -1]`` from ``:150-168``),
* ``FusedTensorProductOp3`` / ``FusedTensorProductOp4`` (``primitives/segmented_polynomial_fused_tp.py:27-75``),
* ``TriMulPrecision`` and ``triangle_multiplicative_update`` (``primitives/triangle.py:20, 238-262``).

This module offers exactly those names with the same arguments, all running on the HIP library; a package
``cuequivariance_ops_torch`` for ROCm is ``from cuequivariance_amd.ops_torch import *`` plus ``register_ops()``.
``register_ops()`` defines ``torch.ops.cuequivariance.uniform_1d`` (21 arguments, same order and meaning).
"""

from __future__ import annotations

import importlib
import itertools
import threading
import weakref
from typing import List, Optional, Sequence

import numpy as np
import torch

from . import cue
from .cuet.transpose import _Permute, _permutation
from .cuet.triangle import TriMulPrecision, triangle_multiplicative_update

# (the package re-exports the function ``uniform_1d`` under the submodule's name: ask for the module itself)
_u1d = importlib.import_module(__package__ + ".cuet.uniform_1d")

__all__ = [
    "uniform_1d",
    "register_ops",
    "segmented_transpose",
    "FusedTensorProductOp3",
    "FusedTensorProductOp4",
    "TriMulPrecision",
    "triangle_multiplicative_update",
]


class uniform_1d:
    """The four batch-mode integers the frontend imports (``segmented_polynomial_uniform_1d.py:25-30``)."""

    BATCH_DIM_AUTO = _u1d.BATCH_DIM_AUTO
    BATCH_DIM_SHARED = _u1d.BATCH_DIM_SHARED
    BATCH_DIM_BATCHED = _u1d.BATCH_DIM_BATCHED
    BATCH_DIM_INDEXED = _u1d.BATCH_DIM_INDEXED


UNIFORM_1D_SCHEMA = (
    "uniform_1d(str name, ScalarType math_dtype, int operand_extent, int num_inputs, int num_outputs, "
    "int num_index, int[] buffer_dim, int[] buffer_num_segments, int[] batch_dim, int[] index_buffer, "
    "int[] dtypes, int num_operations, int[] num_operands, int[] operations, int[] num_paths, "
    "int[] path_indices_start, int[] path_coefficients_start, int[] path_indices, "
    "float[] path_coefficients, int batch_size, Tensor[] tensors) -> Tensor[]"
)

_registered = None
_register_lock = threading.Lock()


def register_ops() -> None:
    """Define ``torch.ops.cuequivariance.uniform_1d`` once per process.  The implementation sits above autograd
    (it is differentiable to any order by re-entering itself with the transposed tables)."""
    global _registered
    with _register_lock:
        if _registered is not None:
            return
        lib = torch.library.Library("cuequivariance", "DEF")
        lib.define(UNIFORM_1D_SCHEMA)
        lib.impl("uniform_1d", _u1d.uniform_1d, "CompositeImplicitAutograd")
        _registered = lib  # the definitions live as long as this object


# ------------------------------------------------------------------------------------------------
# segmented transpose
# ------------------------------------------------------------------------------------------------
_transpose_tables: dict = {}


_transpose_by_address: dict = {}


def _tables_for_info(info: torch.Tensor, device: torch.device):
    # the frontend passes the same registered buffer on every call: recognise it by address and version, so that only
    # the first call reads the table back to the host
    # (tensors made under torch.inference_mode() have no version counter: they are read back on every call)
    if info.is_inference():
        return _tables_for_rows(tuple(map(tuple, info.cpu().to(torch.int64).tolist())), device)
    fast = (info.data_ptr(), info._version, tuple(info.shape), device.type, device.index)
    entry = _transpose_by_address.get(fast)
    if entry is not None and entry[0]() is info:
        return entry[1]
    hit = _tables_for_rows(tuple(map(tuple, info.detach().cpu().to(torch.int64).tolist())), device)
    if len(_transpose_by_address) >= 64:
        _transpose_by_address.pop(next(iter(_transpose_by_address)))
    _transpose_by_address[fast] = (weakref.ref(info), hit)
    return hit


def _tables_for_rows(rows: tuple, device: torch.device):
    key = (rows, device.type, device.index)
    hit = _transpose_tables.get(key)
    if hit is None:
        segments, off = [], 0
        for r in rows:
            if len(r) < 3 or r[0] != off:
                raise ValueError("segmented_transpose: info rows must be [offset, u, v, -1] with running offsets")
            segments.append((int(r[1]), int(r[2])))
            off += int(r[1]) * int(r[2])
        fwd = _permutation(segments)
        bwd = np.empty_like(fwd)
        bwd[fwd] = np.arange(fwd.size, dtype=np.int32)
        hit = (torch.from_numpy(fwd).to(device), torch.from_numpy(bwd).to(device), off)
        if len(_transpose_tables) >= 64:  # a model has a handful of layouts; keep the cache from growing without bound
            _transpose_tables.pop(next(iter(_transpose_tables)))
        _transpose_tables[key] = hit
    return hit


def segmented_transpose(x: torch.Tensor, info: torch.Tensor, contiguous: bool = True) -> torch.Tensor:
    """Every ``(u, v)`` segment of the last axis becomes ``(v, u)``; ``info`` is the frontend's int table
    (``primitives/transpose.py:150-168``).  The result is always a new contiguous tensor."""
    fwd, bwd, total = _tables_for_info(info, x.device)
    if x.shape[-1] != total:
        raise ValueError(f"segmented_transpose: last dimension must be {total}, got {x.shape[-1]}")
    return _Permute.apply(x, fwd, bwd)


# ------------------------------------------------------------------------------------------------
# fused tensor products
# ------------------------------------------------------------------------------------------------
class _FusedTensorProductOp(torch.nn.Module):
    """Callable built from the frontend's description of one descriptor (``segmented_polynomial_fused_tp.py:32-48``):
    subscripts per operand, segment offsets and shapes per operand, path indices ``(P, num_operands)`` and the
    stacked coefficients; the last operand is the output.  Runs the MFMA executor of this engine and raises
    ``NotImplementedError`` for contraction forms it does not cover, like the reference."""

    NUM_OPERANDS = 0

    def __init__(self, operand_segment_modes: Sequence[str], operand_segment_offsets, operand_segment_shapes,
                 path_indices, path_coefficients, math_dtype: Optional[torch.dtype] = None):
        super().__init__()
        from .cuet.segmented_polynomial import SegmentedPolynomial

        modes = [str(m) for m in operand_segment_modes]
        if len(modes) != self.NUM_OPERANDS:
            raise ValueError(f"expected {self.NUM_OPERANDS} operands, got {len(modes)}")
        coeffs = np.asarray(path_coefficients, dtype=np.float64)
        indices = np.asarray(path_indices, dtype=np.int64).reshape(-1, len(modes))
        coeff_modes = ""
        if coeffs.ndim > 1:
            raise NotImplementedError("coefficient modes are not supported by the fused executor")
        d = cue.SegmentedTensorProduct.from_subscripts(",".join(modes) + ("+" + coeff_modes if coeff_modes else ""))
        for oid, (offsets, shapes) in enumerate(zip(operand_segment_offsets, operand_segment_shapes)):
            expect = 0
            for off, shape in zip(offsets, shapes):
                if int(off) != expect:
                    raise ValueError("segments must be packed in order")
                d.add_segment(oid, tuple(int(s) for s in shape))
                expect += int(np.prod(shape)) if len(shape) else 1
        for idx, c in zip(indices, coeffs):
            d.add_path(*[int(i) for i in idx], c=float(c))
        # the frontend hands the inputs over in any order ("u_v_uvw_w", "u_uv_v", ...: ``:117-131``); the executor wants
        # the weights first, so look for the order of the inputs that it accepts
        self.f, self.order = None, None
        n_in = len(modes) - 1
        refusal = None
        for order in itertools.permutations(range(n_in)):
            dd = d.permute_operands(list(order) + [n_in])
            try:
                self.f = SegmentedPolynomial(cue.SegmentedPolynomial.eval_last_operand(dd), method="fused_tp", math_dtype=math_dtype)
            except NotImplementedError as e:
                refusal = e
                continue
            self.order = order
            break
        if self.f is None:
            raise NotImplementedError(f"Fused TP does not support {d.subscripts}: {refusal}")

    def _call(self, inputs: List[torch.Tensor]) -> torch.Tensor:
        return self.f([inputs[k] for k in self.order])[0]


class FusedTensorProductOp3(_FusedTensorProductOp):
    NUM_OPERANDS = 3

    def forward(self, in0: torch.Tensor, in1: torch.Tensor) -> torch.Tensor:
        return self._call([in0, in1])


class FusedTensorProductOp4(_FusedTensorProductOp):
    NUM_OPERANDS = 4

    def forward(self, in0: torch.Tensor, in1: torch.Tensor, in2: torch.Tensor) -> torch.Tensor:
        return self._call([in0, in1, in2])
