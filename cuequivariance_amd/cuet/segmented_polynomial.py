"""``SegmentedPolynomial``: torch module that executes a segmented polynomial on the GPU.

Mirror of ``cuequivariance_torch/cuequivariance_torch/primitives/segmented_polynomial.py:45-372``
(dispatcher: argument checks, choice of method) and of the table builder
``.../segmented_polynomial_uniform_1d.py:82-316``.  Differences:

* every method runs hand-written HIP kernels; there is no PyTorch ("naive") executor in
  this package and no silent fallback.  ``method="naive"`` raises.
* ``method="fused_tp"`` is served by the dense (MFMA) executor when the polynomial has one
  of the supported dense forms, see ``dense.py``.
"""

from __future__ import annotations

import warnings
from typing import Any, Dict, List, Optional

import torch
import torch.nn as nn

from .. import cue
from ..tables import U1dTables
from . import uniform_1d as u1d
from .script import scriptable

__all__ = ["SegmentedPolynomial", "SegmentedPolynomialFromUniform1d"]


def _resolve_math_dtype(math_dtype, method: str):
    if isinstance(math_dtype, str):
        try:
            math_dtype = getattr(torch, math_dtype)
        except AttributeError:
            raise ValueError(
                f"Invalid math_dtype '{math_dtype}' for method '{method}'. Expected 'float32', 'float64', or None."
            )
    if math_dtype not in (None, torch.float32, torch.float64):
        raise ValueError(f"For method '{method}', math_dtype must be 'float32', 'float64', or None; got {math_dtype}")
    return math_dtype


class SegmentedPolynomialFromUniform1d(nn.Module):
    """Flattens a polynomial to scalar coefficients and one uniform mode, builds the flat path tables."""

    def __init__(
        self,
        polynomial: cue.SegmentedPolynomial,
        math_dtype=None,
        output_dtype_map: Optional[List[int]] = None,
        name: str = "segmented_polynomial",
        options: Optional[Dict[str, Any]] = None,
    ):
        super().__init__()
        self._polynomial_orig = polynomial
        self._output_dtype_map_orig = output_dtype_map
        self._options_orig = options

        try:
            polynomial = polynomial.flatten_coefficient_modes()
        except ValueError as e:
            raise ValueError(
                "Failed to prepare polynomial for method 'uniform_1d': this method does not support "
                "coefficient modes and automatic flattening with 'flatten_coefficient_modes()' failed.\n"
                f"Original error:\n{e}\nProblematic polynomial:\n{polynomial}"
            ) from e
        polynomial = polynomial.squeeze_modes()

        for o in polynomial.operands:
            torch._assert(o.ndim in [0, 1], "For method 'uniform_1d', only 0D (scalar) or 1D operands are supported.")
            torch._assert(
                o.all_same_segment_shape(),
                "For method 'uniform_1d', all segments of a given operand must have the same shape. "
                "If segment extents differ but share a common divisor, preprocess the polynomial with "
                "'split_mode()' to obtain uniform segment extents.",
            )
        for ope, stp in polynomial.operations:
            torch._assert(stp.num_operands == len(ope.buffers), "operation/operand count mismatch")
            torch._assert(
                stp.coefficient_subscripts == "",
                "In method 'uniform_1d', coefficients must be scalar (coefficient_subscripts must be empty).",
            )
        try:
            tables = U1dTables.from_polynomial(polynomial, output_dtype_map)
        except ValueError as e:
            raise ValueError(f"For method 'uniform_1d': {e}") from e
        groups = (options or {}).get("segment_groups")
        if groups:
            # {operand: sizes of consecutive groups of its segments}: the rows of that operand are stored channel-major
            # inside every group (an irreps operand in the mul_ir layout, one group per block), and the kernels address
            # them so - no transposition pass around the call.  Not part of the reference's options.
            try:
                tables = tables.with_layouts({int(b): [int(d) for d in dims] for b, dims in groups.items()})
            except ValueError as e:
                raise ValueError(f"For method 'uniform_1d', option 'segment_groups': {e}") from e
        self.tables = tables
        self.num_inputs = polynomial.num_inputs
        self.num_outputs = polynomial.num_outputs
        self.name = name
        self.math_dtype = _resolve_math_dtype(math_dtype, "uniform_1d")
        # the flat lists, under the reference's attribute names
        self.operand_extent = tables.operand_extent
        self.buffer_dim = list(tables.buffer_dim)
        self.buffer_num_segments = list(tables.buffer_num_segments)
        self.dtypes = list(tables.dtypes)
        self.num_operations = len(tables.num_operands)
        self.num_operands = list(tables.num_operands)
        self.operations = list(tables.operations)
        self.num_paths = list(tables.num_paths)
        self.path_indices_start = list(tables.path_indices_start)
        self.path_coefficients_start = list(tables.path_coefficients_start)
        self.path_indices = list(tables.path_indices)
        self.path_coefficients = list(tables.path_coefficients)

        self.BATCH_DIM_AUTO = u1d.BATCH_DIM_AUTO
        self.BATCH_DIM_SHARED = u1d.BATCH_DIM_SHARED
        self.BATCH_DIM_BATCHED = u1d.BATCH_DIM_BATCHED
        self.BATCH_DIM_INDEXED = u1d.BATCH_DIM_INDEXED
        # both math types up front (host-side tables only; device plans are made at the first launch), so that a
        # traced forward only reads this dictionary
        self._plans: dict = {dt: u1d.Uniform1dPlan(self.tables, dt, name=self.name) for dt in (torch.float32, torch.float64)}
        for plan in self._plans.values():
            plan.polynomial = polynomial  # (lets kernels for symmetric contractions be generated at first use)
            plan.origin = (options or {}).get("origin")  # (the descriptor a flattened fully connected product came from)

    def __reduce__(self):
        return (
            SegmentedPolynomial,
            (self._polynomial_orig, "uniform_1d", self.math_dtype, self._output_dtype_map_orig, self.name,
             self._options_orig),
        )

    def _plan(self, math_dtype: torch.dtype) -> u1d.Uniform1dPlan:
        plan = self._plans.get(math_dtype)
        if plan is None:
            plan = u1d.Uniform1dPlan(self.tables, math_dtype, name=self.name)
            self._plans[math_dtype] = plan
        return plan

    def forward(
        self,
        inputs: List[torch.Tensor],
        input_indices: Dict[int, torch.Tensor],
        output_shapes: Dict[int, torch.Tensor],
        output_indices: Dict[int, torch.Tensor],
    ):
        num_index = 0
        batch_dim = [self.BATCH_DIM_AUTO] * (self.num_inputs + self.num_outputs)
        index_buffer = [-1] * (self.num_inputs + self.num_outputs)
        tensors = list(inputs)

        if self.math_dtype is None:
            math_dtype = inputs[0].dtype if inputs[0].dtype in (torch.float32, torch.float64) else torch.float32
        else:
            math_dtype = self.math_dtype

        for pos, idx in input_indices.items():
            batch_dim[pos] = self.BATCH_DIM_INDEXED
            tensors.append(idx)
            index_buffer[pos] = num_index
            num_index += 1
            index_buffer.append(inputs[pos].shape[0])
        for pos, idx in output_indices.items():
            batch_dim[pos + self.num_inputs] = self.BATCH_DIM_INDEXED
            tensors.append(idx)
            index_buffer[pos + self.num_inputs] = num_index
            num_index += 1
            torch._assert(pos in output_shapes, "output shapes must be provided for output indices")
            index_buffer.append(output_shapes[pos].size(0))
        batch_size = self.BATCH_DIM_AUTO
        for pos, shape in output_shapes.items():
            if batch_dim[pos + self.num_inputs] == self.BATCH_DIM_AUTO:
                if shape.size(0) == 1:
                    batch_dim[pos + self.num_inputs] = self.BATCH_DIM_SHARED
                else:
                    torch._assert(
                        batch_size == self.BATCH_DIM_AUTO or batch_size == shape.size(0),
                        "batch size must be auto or the output shape",
                    )
                    batch_dim[pos + self.num_inputs] = self.BATCH_DIM_BATCHED
                    batch_size = shape.size(0)
        # Same data as the 21-argument operator call; the tables are already compiled into a plan.
        return u1d.run_plan(self._plan(math_dtype), batch_dim, index_buffer, batch_size, num_index, tensors)


@scriptable("polynomial")
class SegmentedPolynomial(nn.Module):
    """Executes a ``cue.SegmentedPolynomial`` on tensors of shape ``(batch | 1 | index range, operand_size)``.

    Args:
        polynomial: the descriptor.
        method: ``"uniform_1d"`` (single uniform mode, scalar coefficients after flattening) or
            ``"fused_tp"`` (dense 3-/4-operand contractions).  ``""`` defaults to ``"uniform_1d"`` with a
            warning, as in the reference.
        math_dtype: ``torch.float32``/``torch.float64`` (or their names); default: the input dtype if it is
            one of those, else float32.
        output_dtype_map: for each output, the input whose dtype it inherits (-1: math dtype).
    """

    def __init__(
        self,
        polynomial: cue.SegmentedPolynomial,
        method: str = "",
        math_dtype=None,
        output_dtype_map: Optional[List[int]] = None,
        name: str = "segmented_polynomial",
        options: Optional[Dict[str, Any]] = None,
    ):
        super().__init__()
        self._polynomial_orig = polynomial
        self._math_dtype_orig = math_dtype
        self._output_dtype_map_orig = output_dtype_map
        self.options = options if options is not None else {}
        if not isinstance(polynomial, cue.SegmentedPolynomial):
            raise ValueError(
                f"The polynomial is not a cue.SegmentedPolynomial, but a {type(polynomial)}",
                "Did you forget to call `.polynomial` on the descriptor?",
            )
        self.num_inputs = polynomial.num_inputs
        self.num_outputs = polynomial.num_outputs
        self.repr = repr(polynomial)
        if method == "":
            warnings.warn(
                "SegmentedPolynomial() was called without `method`; defaulting to 'uniform_1d'. "
                "Available methods: 'uniform_1d', 'fused_tp', 'indexed_linear'."
            )
            method = "uniform_1d"
        if method == "uniform_1d":
            self.m = SegmentedPolynomialFromUniform1d(polynomial, math_dtype, output_dtype_map, name, self.options)
        elif method == "fused_tp":
            from .fused_tp import SegmentedPolynomialFusedTP

            # option "rows": "mul_ir" - the irreps operands of a Linear-like polynomial keep the component index contiguous
            # inside every block and the dense kernels address them so (not part of the reference's options)
            self.m = SegmentedPolynomialFusedTP(polynomial, math_dtype, output_dtype_map, name, rows=self.options.get("rows", "ir_mul"),
                                                row_blocks=self.options.get("row_blocks"))
        elif method == "naive":
            raise ValueError(
                "method='naive' (the PyTorch executor) is not part of this engine: every method runs HIP kernels. "
                "Use 'uniform_1d' or 'fused_tp'."
            )
        elif method == "indexed_linear":
            from .dense import SegmentedPolynomialDense

            if math_dtype is not None:
                warnings.warn("`indexed_linear` does not support explicit `math_dtype`.This will be ignored.")
            self.m = SegmentedPolynomialDense(polynomial, None, output_dtype_map, name, method="indexed_linear")
        else:
            raise ValueError(f"Invalid method: {method}")
        self.method = method

    def __reduce__(self):
        return (
            SegmentedPolynomial,
            (self._polynomial_orig, self.method, self._math_dtype_orig, self._output_dtype_map_orig,
             "segmented_polynomial", self.options),
        )

    def __repr__(self):
        return self.repr + f"\n{super().__repr__()}"

    def forward(
        self,
        inputs: List[torch.Tensor],
        input_indices: Optional[Dict[int, torch.Tensor]] = None,
        output_shapes: Optional[Dict[int, torch.Tensor]] = None,
        output_indices: Optional[Dict[int, torch.Tensor]] = None,
    ):
        input_indices = dict(input_indices or {})
        output_shapes = dict(output_shapes or {})
        output_indices = dict(output_indices or {})
        inputs = list(inputs)
        torch._assert(
            len(inputs) == self.num_inputs, "the number of inputs must match the number of inputs of the polynomial"
        )
        for k, v in input_indices.items():
            torch._assert(0 <= k < self.num_inputs, "input index must be in range")
            torch._assert(v.ndim == 1, "input index must be one-dimensional")
            torch._assert(v.dtype in [torch.int32, torch.int64], "input index must be integral")
        for k, v in output_indices.items():
            torch._assert(0 <= k < self.num_outputs, "output index must be in range")
            torch._assert(v.ndim == 1, "input index must be one-dimensional")
            torch._assert(v.dtype in [torch.int32, torch.int64], "input index must be integral")
        for k, v in output_shapes.items():
            torch._assert(0 <= k < self.num_outputs, "output index must be in range")
            torch._assert(v.ndim == 2, "output shape must be two-dimensional")
        return self.m(inputs, input_indices, output_shapes, output_indices)
