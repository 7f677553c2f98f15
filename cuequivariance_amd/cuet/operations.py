"""High-level equivariant layers: channel-wise and fully-connected tensor products, linear.

Constructor arguments, attributes (``irreps_*``, ``weight_numel``, ``weight``, ``shared_weights``,
``internal_weights``, ``method``) and ``forward`` signatures mirror

* ``cuequivariance_torch/cuequivariance_torch/operations/tp_channel_wise.py:30-258``
* ``cuequivariance_torch/cuequivariance_torch/operations/tp_fully_connected.py:30-207``
* ``cuequivariance_torch/cuequivariance_torch/operations/linear.py:30-191``
* ``cuequivariance_torch/cuequivariance_torch/operations/symmetric_contraction.py:32-242``
* ``cuequivariance_torch/cuequivariance_torch/operations/spherical_harmonics.py:26-93``

Defaults differ where the reference defaults to its PyTorch executor: every layer here runs HIP
kernels (``uniform_1d`` for the channel-wise product, the dense executor ``fused_tp`` for the other two).
"""

from __future__ import annotations

import math
import warnings
from typing import Dict, List, Optional, Sequence

import torch

from .. import cue
from ..cue import descriptors
from .script import scriptable
from .segmented_polynomial import SegmentedPolynomial
from .transpose import TransposeIrrepsLayout, apply_layout

__all__ = ["ChannelWiseTensorProduct", "FullyConnectedTensorProduct", "Linear", "SymmetricContraction", "SphericalHarmonics",
           "Rotation", "Inversion", "encode_rotation_angle", "vector_to_euler_angles"]


def _default_irreps(*irreps_list):
    out = []
    for irreps in irreps_list:
        if isinstance(irreps, str):
            irreps = cue.Irreps(irreps)
        elif not isinstance(irreps, cue.Irreps):
            irreps = cue.Irreps(irreps)
        out.append(irreps)
    return tuple(out)


def _assert_same_group(*irreps_list):
    g = irreps_list[0].irrep_class
    for irreps in irreps_list[1:]:
        if irreps.irrep_class is not g:
            raise ValueError("The provided irreps are not of the same group.")


def _transposition_moves(irreps) -> bool:
    """Whether mul_ir and ir_mul differ for these irreps (some block has both a multiplicity and a dimension above one)."""
    return any(mul > 1 and ir.dim > 1 for mul, ir in irreps)


def _default_layout(layout) -> cue.IrrepsLayout:
    if layout is None:
        assumed = cue.get_layout_scope(raising=False)  # (inside ``with cue.assume(layout):``)
        if assumed is not None:
            return assumed
        warnings.warn("layout is not specified, defaulting to cue.mul_ir (the e3nn layout)")
        return cue.mul_ir
    return cue.IrrepsLayout.as_layout(layout)


def _method_from_fallback(method, use_fallback, default: str) -> str:
    if method is not None:
        return method
    if use_fallback is None:
        return default
    warnings.warn("`use_fallback` is deprecated, please use `method` instead", DeprecationWarning)
    if use_fallback:
        raise ValueError("use_fallback=True asks for the PyTorch executor, which this engine does not have")
    return default


class _FlattenedUniform(torch.nn.Module):
    """The same polynomial with every mode but the output's last one flattened away (and that one split down to a
    common extent), which the uniform-1d kernels take.  The dense executor wants one weight row shared by the batch (or
    rows sorted by class); weights per sample or picked by an arbitrary class index are ordinary batched / indexed
    operands here.  Built on first use."""

    def __init__(self, polynomial: cue.SegmentedPolynomial, math_dtype):
        super().__init__()
        self._polynomial, self._math_dtype = polynomial, math_dtype
        self.f = None

    def forward(self, inputs: List[torch.Tensor], input_indices: Optional[Dict[int, torch.Tensor]] = None,
                output_shapes: Optional[Dict[int, torch.Tensor]] = None, output_indices: Optional[Dict[int, torch.Tensor]] = None):
        if self.f is None:
            q = self._polynomial.flatten_coefficient_modes()
            stp = q.operations[0][1]
            keep = stp.subscripts.operands[-1][-1]
            q = q.flatten_modes([m for m in stp.subscripts.modes() if m != keep])
            extents = sorted(q.operations[0][1].get_dims(keep))
            if len(extents) > 1:
                q = q.split_mode(keep, math.gcd(*extents))
            self.f = SegmentedPolynomial(q, method="uniform_1d", math_dtype=self._math_dtype, options={"origin": self._polynomial})
        return self.f(inputs, input_indices=input_indices or {}, output_shapes=output_shapes or {},
                      output_indices=output_indices or {})


@scriptable("with_weight")
class ChannelWiseTensorProduct(torch.nn.Module):
    """``out[k u v] = w[u v] * sum_ij C[i j k] x1[i u] x2[j v]`` for every allowed irrep triple.

    ``forward(x1, x2, weight=None, indices_1=None, indices_2=None, indices_out=None, size_out=None)``:
    ``indices_1`` / ``indices_2`` gather rows of ``x1`` / ``x2`` per batch element, ``indices_out`` scatter-adds
    the batch elements into ``size_out`` output rows.  The forward sums each output row's batch elements in batch
    order (bit-reproducible).  In the backward, the gradient of a gathered operand (``x1`` with ``indices_1``) is
    scattered with floating-point atomics by default - summation order, hence the last bits, vary from run to run; set
    ``CUEQ_DETERMINISTIC=1`` (or ``cuequivariance_amd._lib.set_option("deterministic", 1)``, the C entry point ``cueq_set_option``) for an ordered, bit-reproducible sum at the
    price of one more pass.  The other gradients are bit-reproducible in both modes.
    """

    def __init__(
        self,
        irreps_in1: cue.Irreps,
        irreps_in2: cue.Irreps,
        filter_irreps_out: Sequence[cue.Irrep] = None,
        *,
        layout: Optional[cue.IrrepsLayout] = None,
        layout_in1: Optional[cue.IrrepsLayout] = None,
        layout_in2: Optional[cue.IrrepsLayout] = None,
        layout_out: Optional[cue.IrrepsLayout] = None,
        shared_weights: bool = True,
        internal_weights: bool = None,
        device: Optional[torch.device] = None,
        dtype: Optional[torch.dtype] = None,
        math_dtype=None,
        use_fallback: Optional[bool] = None,
        method: Optional[str] = None,
    ):
        super().__init__()
        irreps_in1, irreps_in2 = _default_irreps(irreps_in1, irreps_in2)
        _assert_same_group(irreps_in1, irreps_in2)
        e = descriptors.channelwise_tensor_product(irreps_in1, irreps_in2, filter_irreps_out)
        descriptor, irreps_out = e.polynomial.operations[0][1], e.outputs[0].irreps
        assert descriptor.subscripts == "uv,iu,jv,kuv+ijk"
        e2 = e.flatten_coefficient_modes().squeeze_modes()
        u1d_compatible = (
            e2.all_same_segment_shape() and len(e2.polynomial.operations[0][1].subscripts.modes()) == 1
        )
        self.irreps_in1, self.irreps_in2, self.irreps_out = irreps_in1, irreps_in2, irreps_out
        self.weight_numel = descriptor.operands[0].size
        self.shared_weights = shared_weights
        self.internal_weights = internal_weights if internal_weights is not None else shared_weights
        if self.internal_weights:
            if not self.shared_weights:
                raise ValueError("Internal weights should be shared")
            self.weight = torch.nn.Parameter(torch.randn(1, self.weight_numel, device=device, dtype=dtype))
        else:
            self.weight = None
        self.method = _method_from_fallback(method, use_fallback, "uniform_1d")
        if self.method == "uniform_1d" and not u1d_compatible:
            raise ValueError(
                "`uniform_1d` method requires segments to be the same shape\n"
                "You can consider making the segments uniform in the descriptor."
            )
        source_in1, target_out = _default_layout(layout_in1 or layout), _default_layout(layout_out or layout)
        # x1 and the output in the mul_ir layout are addressed as they lie by the uniform-1d kernels (the flattened
        # descriptor has one segment per component of a block: a group of ir.dim segments stored channel-major), which
        # saves the transposition pass before and after the product, and their counterparts in the backward
        groups = {}
        if self.method == "uniform_1d":
            if source_in1 == cue.mul_ir and e.inputs[1].layout == cue.ir_mul and _transposition_moves(e.inputs[1].irreps):
                groups[1] = [ir.dim for _, ir in e.inputs[1].irreps]
                source_in1 = cue.ir_mul
            if target_out == cue.mul_ir and e.outputs[0].layout == cue.ir_mul and _transposition_moves(irreps_out):
                groups[3] = [ir.dim for _, ir in irreps_out]
                target_out = cue.ir_mul
        self.transpose_in1 = TransposeIrrepsLayout(e.inputs[1].irreps, source=source_in1, target=e.inputs[1].layout, device=device)
        self.transpose_in2 = TransposeIrrepsLayout(
            e.inputs[2].irreps, source=_default_layout(layout_in2 or layout), target=e.inputs[2].layout, device=device
        )
        self.transpose_out = TransposeIrrepsLayout(irreps_out, source=e.outputs[0].layout, target=target_out, device=device)
        self.f = SegmentedPolynomial(
            e.polynomial, method=self.method, math_dtype=math_dtype, options={"segment_groups": groups} if groups else None
        )

    def extra_repr(self) -> str:
        return (
            f"shared_weights={self.shared_weights}, internal_weights={self.internal_weights}, "
            f"weight_numel={self.weight_numel}"
        )

    def forward(
        self,
        x1: torch.Tensor,
        x2: torch.Tensor,
        weight: Optional[torch.Tensor] = None,
        indices_1: Optional[torch.Tensor] = None,
        indices_2: Optional[torch.Tensor] = None,
        indices_out: Optional[torch.Tensor] = None,
        size_out: Optional[int] = None,
    ) -> torch.Tensor:
        """Arguments as in the reference (``operations/tp_channel_wise.py:186-258``).  Row ids outside ``[0, size_out)`` in ``indices_out`` raise an error in eager mode; while the current stream is being
        captured into a HIP graph the grouping of the batch rows by output row is recorded as device work that cannot report
        them: such batch rows are left out of every output row, at capture and at every replay."""
        x1 = apply_layout(self.transpose_in1, x1)
        x2 = apply_layout(self.transpose_in2, x2)
        indices_in: Dict[int, torch.Tensor] = {}
        if indices_1 is not None:
            indices_in[1] = indices_1
        if indices_2 is not None:
            indices_in[2] = indices_2
        indices_o: Dict[int, torch.Tensor] = {}
        sizes_out: Dict[int, torch.Tensor] = {}
        if indices_out is not None:
            if size_out is None:
                raise ValueError("size_out should be provided if indices_out is provided")
            indices_o = {0: indices_out}
            sizes_out = {0: torch.empty(size_out, 1, device="meta")}  # only .shape[0] is read
        if self.weight is not None:
            if weight is not None:
                raise ValueError("Internal weights are used, weight should be None")
            weight = self.weight
        elif weight is None:
            raise ValueError("Internal weights are not used, weight should not be None")
        out = self.f([weight, x1, x2], input_indices=indices_in, output_shapes=sizes_out, output_indices=indices_o)
        return apply_layout(self.transpose_out, out[0])


class ChannelWiseSphericalTensorProduct(torch.nn.Module):
    """``ChannelWiseTensorProduct(irreps_in1, Y_ls, filter)(x1, SphericalHarmonics(ls, normalize)(vectors), weight, ...)`` as one
    polynomial of ``(weight, x1, vectors)``: the harmonics of the edge vectors are evaluated in registers inside the edge
    kernels - they are neither written nor read back - and the backward returns the gradient with respect to the vectors.
    An extension over the reference, which runs the two modules one after the other
    (``cuequivariance_torch/operations/spherical_harmonics.py:26-93``, ``tp_channel_wise.py:30-258``).

    ``forward(x1, vectors (batch, 3), weight=None, indices_1=None, indices_out=None, size_out=None)``; weights, irreps of the
    output, layouts and indices as for ``ChannelWiseTensorProduct``; component normalisation of the harmonics,
    ``normalize=True`` divides the vectors by their norm first (as ``SphericalHarmonics`` does).
    """

    def __init__(
        self,
        irreps_in1: cue.Irreps,
        ls: Sequence[int],
        filter_irreps_out: Sequence[cue.Irrep] = None,
        *,
        normalize: bool = True,
        layout: Optional[cue.IrrepsLayout] = None,
        layout_in1: Optional[cue.IrrepsLayout] = None,
        layout_out: Optional[cue.IrrepsLayout] = None,
        shared_weights: bool = True,
        internal_weights: bool = None,
        device: Optional[torch.device] = None,
        dtype: Optional[torch.dtype] = None,
        math_dtype=None,
    ):
        super().__init__()
        from ..cue import fused

        ls = list(ls)
        if ls != sorted(set(ls)) or not ls:
            raise ValueError(f"ls must be ascending and unique, got {ls}")
        self.ls, self.normalize = ls, normalize
        polynomial, info, irreps_out = fused.channelwise_spherical(irreps_in1, ls, filter_irreps_out)
        self.irreps_in1, self.irreps_out = irreps_in1, irreps_out
        self.weight_numel = polynomial.inputs[0].size
        self.shared_weights = shared_weights
        self.internal_weights = internal_weights if internal_weights is not None else shared_weights
        if self.internal_weights:
            if not self.shared_weights:
                raise ValueError("Internal weights should be shared")
            self.weight = torch.nn.Parameter(torch.randn(1, self.weight_numel, device=device, dtype=dtype))
        else:
            self.weight = None
        source_in1, target_out = _default_layout(layout_in1 or layout), _default_layout(layout_out or layout)
        groups = {}
        if source_in1 == cue.mul_ir and _transposition_moves(irreps_in1):
            groups[1] = [ir.dim for _, ir in irreps_in1]
            source_in1 = cue.ir_mul
        if target_out == cue.mul_ir and _transposition_moves(irreps_out):
            groups[3] = [ir.dim for _, ir in irreps_out]
            target_out = cue.ir_mul
        self.transpose_in1 = TransposeIrrepsLayout(irreps_in1, source=source_in1, target=cue.ir_mul, device=device)
        self.transpose_out = TransposeIrrepsLayout(irreps_out, source=cue.ir_mul, target=target_out, device=device)
        options = {"origin": info}
        if groups:
            options["segment_groups"] = groups
        self.f = SegmentedPolynomial(polynomial, method="uniform_1d", math_dtype=math_dtype, options=options)

    def extra_repr(self) -> str:
        return f"ls={self.ls}, normalize={self.normalize}, shared_weights={self.shared_weights}, weight_numel={self.weight_numel}"

    def forward(
        self,
        x1: torch.Tensor,
        vectors: torch.Tensor,
        weight: Optional[torch.Tensor] = None,
        indices_1: Optional[torch.Tensor] = None,
        indices_out: Optional[torch.Tensor] = None,
        size_out: Optional[int] = None,
    ) -> torch.Tensor:
        torch._assert(vectors.ndim == 2 and vectors.shape[1] == 3, f"vectors must have shape (batch, 3) - got {vectors.shape}")
        if self.normalize:
            vectors = torch.nn.functional.normalize(vectors, dim=1)
        x1 = apply_layout(self.transpose_in1, x1)
        indices_in: Dict[int, torch.Tensor] = {} if indices_1 is None else {1: indices_1}
        indices_o: Dict[int, torch.Tensor] = {}
        sizes_out: Dict[int, torch.Tensor] = {}
        if indices_out is not None:
            if size_out is None:
                raise ValueError("size_out should be provided if indices_out is provided")
            indices_o = {0: indices_out}
            sizes_out = {0: torch.empty(size_out, 1, device="meta")}  # only .shape[0] is read
        if self.weight is not None:
            if weight is not None:
                raise ValueError("Internal weights are used, weight should be None")
            weight = self.weight
        elif weight is None:
            raise ValueError("Internal weights are not used, weight should not be None")
        out = self.f([weight, x1, vectors], input_indices=indices_in, output_shapes=sizes_out, output_indices=indices_o)
        return apply_layout(self.transpose_out, out[0])


@scriptable("fully_connected")
class FullyConnectedTensorProduct(torch.nn.Module):
    """``out[k w] = sum_{u v i j} w[u v w] C[i j k] x1[i u] x2[j v]`` over every allowed irrep triple."""

    def __init__(
        self,
        irreps_in1: cue.Irreps,
        irreps_in2: cue.Irreps,
        irreps_out: cue.Irreps,
        *,
        layout: Optional[cue.IrrepsLayout] = None,
        layout_in1: Optional[cue.IrrepsLayout] = None,
        layout_in2: Optional[cue.IrrepsLayout] = None,
        layout_out: Optional[cue.IrrepsLayout] = None,
        shared_weights: bool = True,
        internal_weights: bool = None,
        device: Optional[torch.device] = None,
        dtype: Optional[torch.dtype] = None,
        math_dtype=None,
        use_fallback: Optional[bool] = None,
        method: Optional[str] = None,
    ):
        super().__init__()
        irreps_in1, irreps_in2, irreps_out = _default_irreps(irreps_in1, irreps_in2, irreps_out)
        _assert_same_group(irreps_in1, irreps_in2, irreps_out)
        if dtype is None:
            dtype = torch.get_default_dtype()
        e = descriptors.fully_connected_tensor_product(irreps_in1, irreps_in2, irreps_out)
        assert e.polynomial.operations[0][1].subscripts == "uvw,iu,jv,kw+ijk"
        self.irreps_in1, self.irreps_in2, self.irreps_out = irreps_in1, irreps_in2, irreps_out
        self.weight_numel = e.polynomial.operations[0][1].operands[0].size
        self.shared_weights = shared_weights
        self.internal_weights = internal_weights if internal_weights is not None else shared_weights
        if self.internal_weights:
            if not self.shared_weights:
                raise ValueError("Internal weights should be shared")
            self.weight = torch.nn.Parameter(torch.randn(1, self.weight_numel, device=device, dtype=dtype))
        else:
            self.weight = None
        self.transpose_in1 = TransposeIrrepsLayout(
            e.inputs[1].irreps, source=_default_layout(layout_in1 or layout), target=e.inputs[1].layout, device=device
        )
        self.transpose_in2 = TransposeIrrepsLayout(
            e.inputs[2].irreps, source=_default_layout(layout_in2 or layout), target=e.inputs[2].layout, device=device
        )
        self.transpose_out = TransposeIrrepsLayout(
            e.outputs[0].irreps, source=e.outputs[0].layout, target=_default_layout(layout_out or layout), device=device
        )
        self.method = _method_from_fallback(method, use_fallback, "fused_tp")
        self.f_per_sample = _FlattenedUniform(e.polynomial, math_dtype)  # weights of shape (batch, weight_numel)
        self.f = SegmentedPolynomial(e.polynomial, method=self.method, math_dtype=math_dtype)
        if getattr(self.f.m, "dense", True) is None and getattr(self.f.m, "composed", None) is None:
            # the matrix-core executor takes a second operand of multiplicity one directly, any other behind a stage that
            # forms the products of the two operands; what neither takes runs on the uniform-1d kernels of the flattened
            # descriptor, with the weight row shared by the batch
            self.f = None
        # mul_ir rows of the first operand and of the output taken as they lie by the generated fused kernels (no
        # transposition pass) when those kernels serve the call; everything else keeps the passes
        self.f_rows = None
        if (self.f is not None and self.method == "fused_tp" and self.transpose_in1.source == cue.mul_ir
                and self.transpose_out.target == cue.mul_ir and e.inputs[1].layout == cue.ir_mul and e.outputs[0].layout == cue.ir_mul
                and (_transposition_moves(e.inputs[1].irreps) or _transposition_moves(e.outputs[0].irreps))):
            try:
                self.f_rows = SegmentedPolynomial(
                    e.polynomial, method="fused_tp", math_dtype=math_dtype,
                    options={"rows": "mul_ir", "row_blocks": ([(mul, ir.dim) for mul, ir in e.inputs[1].irreps],
                                                               [(mul, ir.dim) for mul, ir in e.outputs[0].irreps])})
            except (NotImplementedError, ValueError):
                self.f_rows = None

    def extra_repr(self) -> str:
        return (
            f"shared_weights={self.shared_weights}, internal_weights={self.internal_weights}, "
            f"weight_numel={self.weight_numel}"
        )

    def forward(self, x1: torch.Tensor, x2: torch.Tensor, weight: Optional[torch.Tensor] = None, *,
                indices_1: Optional[torch.Tensor] = None, indices_out: Optional[torch.Tensor] = None,
                size_out: Optional[int] = None) -> torch.Tensor:
        """``indices_1`` (rows of ``x1`` per batch element) and ``indices_out`` / ``size_out`` (output row per batch
        element, summed) are extensions over the reference's signature: gather and scatter-sum inside the kernel.
        Row ids outside ``[0, size_out)`` in ``indices_out`` raise an error in eager mode; while the current stream is being
        captured into a HIP graph the grouping of the batch rows by output row is recorded as device work that cannot report
        them: such batch rows are left out of every output row, at capture and at every replay."""
        if self.weight is not None:
            if weight is not None:
                raise ValueError("Internal weights are used, weight should be None")
            weight = self.weight
        elif weight is None:
            raise ValueError("Internal weights are not used, weight should not be None")
        if indices_1 is None and indices_out is None and self._rows_ready(x1, x2, weight):
            return self.f_rows([weight, x1, apply_layout(self.transpose_in2, x2)])[0]
        x1 = apply_layout(self.transpose_in1, x1)
        x2 = apply_layout(self.transpose_in2, x2)
        if indices_1 is not None or indices_out is not None:
            if indices_out is not None and size_out is None:
                raise ValueError("size_out should be provided if indices_out is provided")
            out = self.f_per_sample(
                [weight, x1, x2], {} if indices_1 is None else {1: indices_1},
                {} if indices_out is None else {0: torch.empty(size_out, 1, device="meta")},
                {} if indices_out is None else {0: indices_out})
            return apply_layout(self.transpose_out, out[0])
        if weight.shape[0] != 1 or self.f is None:
            return apply_layout(self.transpose_out, self.f_per_sample([weight, x1, x2])[0])
        return apply_layout(self.transpose_out, self.f([weight, x1, x2])[0])

    def _rows_ready(self, x1, x2, weight) -> bool:
        dense = self.f_rows.m.dense if self.f_rows is not None else None
        return (dense is not None and weight is not None and weight.shape[0] == 1 and x1.is_cuda and x1.dtype == x2.dtype == weight.dtype
                and x1.shape[0] == x2.shape[0] and dense.mul_ir_ready(x1.dtype))


@scriptable("linear")
class Linear(torch.nn.Module):
    """Equivariant linear map: one ``mul_in x mul_out`` weight block per pair of equal irreps, scaled ``1/sqrt(mul_in)``.

    ``forward(x, weight=None, weight_indices=None)``; with ``weight_classes > 1`` the weights have one row per
    class and ``weight_indices`` selects the row used by each batch element.
    """

    def __init__(
        self,
        irreps_in: cue.Irreps,
        irreps_out: cue.Irreps,
        *,
        layout: Optional[cue.IrrepsLayout] = None,
        layout_in: Optional[cue.IrrepsLayout] = None,
        layout_out: Optional[cue.IrrepsLayout] = None,
        shared_weights: bool = True,
        internal_weights: bool = None,
        weight_classes: Optional[int] = 1,
        device: Optional[torch.device] = None,
        dtype: Optional[torch.dtype] = None,
        math_dtype=None,
        use_fallback: Optional[bool] = None,
        method: Optional[str] = None,
    ):
        super().__init__()
        irreps_in, irreps_out = _default_irreps(irreps_in, irreps_out)
        _assert_same_group(irreps_in, irreps_out)
        e = descriptors.linear(irreps_in, irreps_out)
        assert e.polynomial.operations[0][1].subscripts == "uv,iu,iv"
        self.irreps_in, self.irreps_out = irreps_in, irreps_out
        self.weight_numel = e.inputs[0].dim
        self.weight_classes = weight_classes
        self.shared_weights = shared_weights
        if weight_classes > 1 and not shared_weights:
            raise ValueError("Weight classes require shared weights.")
        self.internal_weights = internal_weights if internal_weights is not None else shared_weights
        if self.internal_weights:
            if not self.shared_weights:
                raise ValueError("Internal weights should be shared")
            self.weight = torch.nn.Parameter(torch.randn(weight_classes, self.weight_numel, device=device, dtype=dtype))
        else:
            self.weight = None
        self.transpose_in = TransposeIrrepsLayout(
            e.inputs[1].irreps, source=_default_layout(layout_in or layout), target=e.inputs[1].layout, device=device
        )
        self.transpose_out = TransposeIrrepsLayout(
            e.outputs[0].irreps, source=e.outputs[0].layout, target=_default_layout(layout_out or layout), device=device
        )
        self.method = _method_from_fallback(method, use_fallback, "fused_tp")
        self.f = SegmentedPolynomial(e.polynomial, method=self.method, math_dtype=math_dtype)
        # weights per sample, or per class with an index in any order (sorted classes: method="indexed_linear")
        self.f_per_sample = _FlattenedUniform(e.polynomial, math_dtype)
        # mul_ir rows on both sides: the dense kernels address them as they lie (no transposition pass) whenever the blocks
        # have a shape those kernels take; other shapes, dtypes and per-sample / indexed weights keep the passes
        self.f_rows = None
        if (self.method == "fused_tp" and self.transpose_in.source == cue.mul_ir and self.transpose_out.target == cue.mul_ir
                and e.inputs[1].layout == cue.ir_mul and e.outputs[0].layout == cue.ir_mul
                and (_transposition_moves(e.inputs[1].irreps) or _transposition_moves(e.outputs[0].irreps))):
            try:
                self.f_rows = SegmentedPolynomial(e.polynomial, method="fused_tp", math_dtype=math_dtype, options={"rows": "mul_ir"})
            except NotImplementedError:
                self.f_rows = None

    def extra_repr(self) -> str:
        return (
            f"shared_weights={self.shared_weights}, internal_weights={self.internal_weights}, "
            f"weight_numel={self.weight_numel}"
        )

    def forward(
        self, x: torch.Tensor, weight: Optional[torch.Tensor] = None, weight_indices: Optional[torch.Tensor] = None
    ) -> torch.Tensor:
        if self.internal_weights:
            if weight is not None:
                raise ValueError("Internal weights are used, weight should be None")
            weight = self.weight
        input_indices: Dict[int, torch.Tensor] = {}
        if self.weight_classes > 1:
            if weight_indices is None:
                raise ValueError("weight_indices should be provided if weight_classes > 1")
            input_indices[0] = weight_indices
        if weight is None:
            raise ValueError("Weights should not be None")
        if (self.f_rows is not None and not input_indices and weight.shape[0] == 1 and x.is_cuda and x.dtype == weight.dtype
                and self.f_rows.m.dense.mul_ir.accepts(x.dtype)):
            return self.f_rows([weight, x])[0]
        if self.method != "indexed_linear" and (input_indices or weight.shape[0] != 1):
            out = self.f_per_sample([weight, apply_layout(self.transpose_in, x)], input_indices)
        else:
            out = self.f([weight, apply_layout(self.transpose_in, x)], input_indices=input_indices)
        return apply_layout(self.transpose_out, out[0])


@scriptable("contraction")
class SymmetricContraction(torch.nn.Module):
    """Symmetric contraction of MACE (https://arxiv.org/abs/2206.07697): for every degree ``n`` up to
    ``contraction_degree`` the symmetric part of ``x ⊗ ... ⊗ x`` (``n`` factors) is mapped onto ``irreps_out`` with
    one learned weight per independent coupling, channel and element type.

    ``weight`` has shape ``(num_elements, weight_shape[0], mul)``; ``forward(x, indices)`` picks the weight row of each
    batch element by ``indices`` (int32 or int64, one per row of ``x``).  With ``original_mace=True`` the weights are
    those of the original MACE parametrisation and are projected onto the standard basis at every call.
    All multiplicities of ``irreps_in`` and ``irreps_out`` must be equal.
    """

    def __init__(
        self,
        irreps_in: cue.Irreps,
        irreps_out: cue.Irreps,
        contraction_degree: int,
        num_elements: int,
        *,
        layout: Optional[cue.IrrepsLayout] = None,
        layout_in: Optional[cue.IrrepsLayout] = None,
        layout_out: Optional[cue.IrrepsLayout] = None,
        device: Optional[torch.device] = None,
        dtype: Optional[torch.dtype] = None,
        math_dtype=None,
        original_mace: bool = False,
        use_fallback: Optional[bool] = None,
        method: Optional[str] = None,
    ):
        super().__init__()
        irreps_in, irreps_out = _default_irreps(irreps_in, irreps_out)
        _assert_same_group(irreps_in, irreps_out)
        self.contraction_degree = contraction_degree
        if len(set(irreps_in.muls) | set(irreps_out.muls)) != 1:
            raise ValueError("Input/Output irreps must have the same mul")
        mul = irreps_in.muls[0]
        self.irreps_in, self.irreps_out = irreps_in, irreps_out
        self.etp, p = cue.mace.symmetric_contraction(irreps_in, irreps_out, range(1, contraction_degree + 1))
        if original_mace:
            self.register_buffer("projection", torch.tensor(p, dtype=dtype, device=device))
            self.weight_shape = (p.shape[0], mul)
        else:
            self.projection = None
            self.weight_shape = (self.etp.inputs[0].dim // mul, mul)
        self.num_elements = num_elements
        self.weight = torch.nn.Parameter(torch.randn(num_elements, *self.weight_shape, device=device, dtype=dtype))
        if method == "uniform_1d" and not self.etp.polynomial.all_same_segment_shape():
            raise ValueError("`uniform_1d` method requires segments to be the same shape")
        self.method = _method_from_fallback(method, use_fallback, "uniform_1d")
        source_in, target_out = _default_layout(layout_in or layout), _default_layout(layout_out or layout)
        # mul_ir rows of x and of the output are addressed as they lie by the uniform-1d kernels (see ChannelWiseTensorProduct)
        groups = {}
        if self.method == "uniform_1d":
            if source_in == cue.mul_ir and self.etp.inputs[1].layout == cue.ir_mul and _transposition_moves(self.etp.inputs[1].irreps):
                groups[1] = [ir.dim for _, ir in self.etp.inputs[1].irreps]
                source_in = cue.ir_mul
            if target_out == cue.mul_ir and self.etp.outputs[0].layout == cue.ir_mul and _transposition_moves(self.etp.outputs[0].irreps):
                groups[2] = [ir.dim for _, ir in self.etp.outputs[0].irreps]
                target_out = cue.ir_mul
        self.transpose_in = TransposeIrrepsLayout(
            self.etp.inputs[1].irreps, source=source_in, target=self.etp.inputs[1].layout, device=device,
        )
        self.transpose_out = TransposeIrrepsLayout(
            self.etp.outputs[0].irreps, source=self.etp.outputs[0].layout, target=target_out, device=device,
        )
        self.f = SegmentedPolynomial(self.etp.polynomial, method=self.method, math_dtype=math_dtype,
                                     options={"segment_groups": groups} if groups else None)

    def extra_repr(self) -> str:
        return f"contraction_degree={self.contraction_degree}, weight_shape={self.weight_shape}"

    def forward(self, x: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
        """``x``: ``(batch, irreps_in.dim)``; ``indices``: ``(batch,)``; returns ``(batch, irreps_out.dim)``."""
        if self.projection is not None:
            weight = torch.einsum("zau,ab->zbu", self.weight, self.projection)
        else:
            weight = self.weight
        out = self.f([weight.flatten(1), apply_layout(self.transpose_in, x)], input_indices={0: indices})
        return apply_layout(self.transpose_out, out[0])


@scriptable("vectors")
class SphericalHarmonics(torch.nn.Module):
    """Spherical harmonics of 3-vectors: ``forward(vectors (batch, 3)) -> (batch, sum(2l+1))`` for the degrees ``ls``
    (ascending, unique); component normalisation, ``Y_1 = sqrt(3) x``.  ``normalize=True`` divides the vectors by their
    norm first."""

    def __init__(self, ls, normalize: bool = True, device: Optional[torch.device] = None, math_dtype=None,
                 use_fallback: Optional[bool] = None, method: Optional[str] = None):
        super().__init__()
        self.ls = ls if isinstance(ls, list) else [ls]
        assert self.ls == sorted(set(self.ls))
        self.normalize = normalize
        e = descriptors.spherical_harmonics(cue.SO3(1), self.ls)
        self.method = _method_from_fallback(method, use_fallback, "uniform_1d")
        self.f = SegmentedPolynomial(e.polynomial, method=self.method, math_dtype=math_dtype)

    def forward(self, vectors: torch.Tensor) -> torch.Tensor:
        torch._assert(vectors.ndim == 2, f"Input must have shape (batch, 3) - got {vectors.shape}")
        if self.normalize:
            vectors = torch.nn.functional.normalize(vectors, dim=1)
        [output] = self.f([vectors])
        return output


@scriptable("rotation")
class Rotation(torch.nn.Module):
    """Rotation of SO(3) / O(3) features (``cuequivariance_torch/operations/rotation.py:29-157`` in the reference):
    ``forward(gamma, beta, alpha, x)`` applies the rotation about y by ``gamma``, then about x by ``beta``, then about y by
    ``alpha`` to every irrep of ``x`` - ``R = R_y(alpha) R_x(beta) R_y(gamma)``, active and right-handed on the components
    ``(x, y, z)`` of a vector.  Angles: one per row of ``x``, or a single one for all rows.  One uniform-1d polynomial with the three
    angle encodings and ``x`` as inputs (``descriptors.yxy_rotation``)."""

    def __init__(
        self,
        irreps: cue.Irreps,
        *,
        layout: Optional[cue.IrrepsLayout] = None,
        layout_in: Optional[cue.IrrepsLayout] = None,
        layout_out: Optional[cue.IrrepsLayout] = None,
        device: Optional[torch.device] = None,
        math_dtype=None,
        use_fallback: Optional[bool] = None,
        method: Optional[str] = None,
    ):
        super().__init__()
        (irreps,) = _default_irreps(irreps)
        if irreps.irrep_class not in [cue.SO3, cue.O3]:
            raise ValueError(f"Unsupported irrep class {irreps.irrep_class}. Must be SO3 or O3.")
        e = descriptors.yxy_rotation(irreps)
        self.irreps = irreps
        self.lmax = max(ir.l for _, ir in irreps)
        self.transpose_in = TransposeIrrepsLayout(
            e.inputs[3].irreps, source=_default_layout(layout_in or layout), target=e.inputs[3].layout, device=device
        )
        self.transpose_out = TransposeIrrepsLayout(
            e.outputs[0].irreps, source=e.outputs[0].layout, target=_default_layout(layout_out or layout), device=device
        )
        self.method = _method_from_fallback(method, use_fallback, "uniform_1d")
        # (multiplicities that differ: the channel mode split down to their common divisor)
        self.f = (SegmentedPolynomial(e.polynomial, method=self.method, math_dtype=math_dtype)
                  if e.polynomial.all_same_segment_shape() or self.method != "uniform_1d" else _FlattenedUniform(e.polynomial, math_dtype))

    def forward(self, gamma: torch.Tensor, beta: torch.Tensor, alpha: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
        encodings = []
        for angle in (gamma, beta, alpha):
            angle = torch.as_tensor(angle, dtype=x.dtype, device=x.device)
            enc = encode_rotation_angle(angle, self.lmax)
            encodings.append(enc.reshape(-1, enc.shape[-1]))  # (1 or batch, 2 lmax + 1)
        out = self.f([*encodings, apply_layout(self.transpose_in, x)])
        return apply_layout(self.transpose_out, out[0])


def encode_rotation_angle(angle: torch.Tensor, ell: int) -> torch.Tensor:
    """``[cos(ell a), cos((ell - 1) a), ..., cos(a), 1, sin(a), sin(2 a), ..., sin(ell a)]`` along a new last axis: the form in
    which the rotation polynomials take an angle (``operations/rotation.py:160-176`` in the reference)."""
    angle = torch.as_tensor(angle).unsqueeze(-1)
    m = torch.arange(1, ell + 1, device=angle.device, dtype=angle.dtype)
    return torch.cat([torch.cos(m.flip(0) * angle), torch.ones_like(angle), torch.sin(m * angle)], dim=-1)


def vector_to_euler_angles(vector: torch.Tensor):
    """``(beta, alpha)`` with ``R_y(alpha) R_x(beta) e_y = vector / |vector|`` (``operations/rotation.py:179-208`` in the
    reference): ``beta`` is the angle to the y axis, ``alpha`` the azimuth from z towards x (0 on the y axis itself)."""
    assert vector.shape[-1] == 3
    x, y, z = torch.nn.functional.normalize(vector.reshape(-1, 3), dim=-1).unbind(-1)
    on_axis = (x == 0.0) & (z == 0.0)
    beta = torch.acos(torch.clamp(torch.where(on_axis, torch.sign(y), y), -1.0, 1.0))
    alpha = torch.atan2(torch.where(on_axis, torch.zeros_like(x), x), torch.where(on_axis, torch.ones_like(z), z))
    return beta.reshape(vector.shape[:-1]), alpha.reshape(vector.shape[:-1])


@scriptable("x")
class Inversion(torch.nn.Module):
    """Inversion ``x -> -x`` of O(3) features: every irrep times its parity (``operations/rotation.py:211-310`` in the
    reference)."""

    def __init__(
        self,
        irreps: cue.Irreps,
        *,
        layout: Optional[cue.IrrepsLayout] = None,
        layout_in: Optional[cue.IrrepsLayout] = None,
        layout_out: Optional[cue.IrrepsLayout] = None,
        device: Optional[torch.device] = None,
        math_dtype=None,
        use_fallback: Optional[bool] = None,
        method: Optional[str] = None,
    ):
        super().__init__()
        (irreps,) = _default_irreps(irreps)
        if irreps.irrep_class not in [cue.O3]:
            raise ValueError(f"Unsupported irrep class {irreps.irrep_class}. Must be O3.")
        e = descriptors.inversion(irreps)
        self.irreps = irreps
        self.transpose_in = TransposeIrrepsLayout(
            e.inputs[0].irreps, source=_default_layout(layout_in or layout), target=e.inputs[0].layout, device=device
        )
        self.transpose_out = TransposeIrrepsLayout(
            e.outputs[0].irreps, source=e.outputs[0].layout, target=_default_layout(layout_out or layout), device=device
        )
        self.method = _method_from_fallback(method, use_fallback, "uniform_1d")
        self.f = (SegmentedPolynomial(e.polynomial, method=self.method, math_dtype=math_dtype)
                  if e.polynomial.all_same_segment_shape() or self.method != "uniform_1d" else _FlattenedUniform(e.polynomial, math_dtype))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return apply_layout(self.transpose_out, self.f([apply_layout(self.transpose_in, x)])[0])
