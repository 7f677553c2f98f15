"""``method="fused_tp"`` on every contraction form the reference's dispatcher lists
(``cuequivariance_torch/cuequivariance_torch/primitives/segmented_polynomial_fused_tp.py:114-129``), on polynomials with
several operations, and with gathered inputs / scattered outputs (``:186-262``), against the CPU oracle.

Tolerances: float64 ``1e-12 * max|ref|``, float32 ``1e-5 * max|ref|``.
"""

import itertools

import numpy as np
import pytest
import torch

from cuequivariance_amd import cue
from cuequivariance_amd.cue import SegmentedTensorProduct as STP
from oracle.naive import naive_segmented_polynomial, spec_from_polynomial

FORMS = ["u,,uw,w", ",v,vw,w", "u,v,uv,u", "u,v,uv,v", "u,u,uw,w", "u,v,uvw,w", "u,u,u", "u,v,uv", "u,uv,v", "u,,u", ",v,v"]
DIMS = dict(u=8, v=4, w=16)
TOL = {torch.float64: 1e-12, torch.float32: 1e-5}


def random_stp(subscripts: str, seed: int, nseg: int = 2) -> STP:
    d = STP.from_subscripts(subscripts)
    operands = subscripts.split(",")
    for i, o in enumerate(operands):
        for _ in range(nseg):
            d.add_segment(i, tuple(DIMS[m] for m in o))
    rng = np.random.default_rng(seed)
    for idx in itertools.product(range(nseg), repeat=len(operands)):
        if rng.random() < 0.6:
            d.add_path(*idx, c=float(rng.normal()))
    if d.num_paths == 0:
        d.add_path(*([0] * len(operands)), c=1.5)
    return d


def rel_err(got, ref):
    return (got.detach().cpu().double() - ref.double()).abs().max().item() / max(ref.abs().max().item(), 1e-30)


def check(device, poly, inputs, dtype, input_indices=None, output_shapes=None, output_indices=None, expect_dense=None):
    from cuequivariance_amd import cuet

    m = cuet.SegmentedPolynomial(poly, method="fused_tp", math_dtype=dtype)
    if expect_dense is not None:
        assert (m.m.dense is not None) == expect_dense
    spec = spec_from_polynomial(poly)
    a = [t.clone().requires_grad_(True) for t in inputs]
    sizes = {k: v.shape[0] for k, v in (output_shapes or {}).items()}
    ref = naive_segmented_polynomial(spec, a, input_indices or {}, sizes, output_indices or {})
    cots = [torch.randn(r.shape, dtype=torch.float64, generator=torch.Generator().manual_seed(9)).to(dtype) for r in ref]
    ref_grads = torch.autograd.grad(ref, a, cots)
    b = [t.clone().to(device).requires_grad_(True) for t in inputs]
    got = m(b, {k: v.to(device) for k, v in (input_indices or {}).items()},
            {k: torch.empty(v.shape[0], 1, device=device) for k, v in (output_shapes or {}).items()},
            {k: v.to(device) for k, v in (output_indices or {}).items()})
    assert len(got) == len(ref)
    for g_, r_ in zip(got, ref):
        assert g_.dtype == dtype and g_.shape == r_.shape
        assert rel_err(g_, r_) <= TOL[dtype], rel_err(g_, r_)
    grads = torch.autograd.grad(got, b, [c.to(device) for c in cots])
    for g_, r_ in zip(grads, ref_grads):
        assert rel_err(g_, r_) <= TOL[dtype], rel_err(g_, r_)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("form", FORMS)
def test_every_reference_form(device, form, dtype):
    d = random_stp(form, seed=len(form) + sum(map(ord, form)))
    poly = cue.SegmentedPolynomial.eval_last_operand(d)
    g = torch.Generator().manual_seed(1)
    Z = 37
    inputs = [torch.randn(Z, o.size, dtype=torch.float64, generator=g).to(dtype) for o in poly.inputs]
    check(device, poly, inputs, dtype)


@pytest.mark.gpu
def test_linear_with_weights_in_second_position_runs_on_the_matrix_cores(device):
    """``u,uv,v`` is ``uv,u,v`` with its inputs swapped: the wrapper finds the order the matrix-core executor takes."""
    d = random_stp("u,uv,v", seed=4)
    poly = cue.SegmentedPolynomial.eval_last_operand(d)
    g = torch.Generator().manual_seed(2)
    inputs = [torch.randn(301, poly.inputs[0].size, dtype=torch.float64, generator=g).float(),
              torch.randn(1, poly.inputs[1].size, dtype=torch.float64, generator=g).float()]
    check(device, poly, inputs, torch.float32, expect_dense=True)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_several_operations_and_outputs(device, dtype):
    """Two operations add into output 0 (one element-wise ``u,u,u``, one with a shared weight row ``uv,u,v`` read from
    another input), a third writes output 1; inputs 0 and 1 are gathered, output 0 is scattered."""
    a_ = random_stp("u,u,u", seed=11)
    b_ = random_stp("u,uv,v", seed=12)
    # make operand shapes agree: x[u] (2 segments of 8), y[u], w[uv] with v = 8 so that out0 = 2 segments of 8
    dims = dict(DIMS)
    DIMS.update(v=8)
    try:
        b_ = random_stp("u,uv,v", seed=12)
        c_ = random_stp("u,,u", seed=13)
    finally:
        DIMS.clear()
        DIMS.update(dims)
    x, y, w, s, out0, out1 = a_.operands[0], a_.operands[1], b_.operands[1], c_.operands[1], a_.operands[2], c_.operands[2]
    assert b_.operands[0] == x and b_.operands[2] == out0 and c_.operands[0] == x
    poly = cue.SegmentedPolynomial([x, y, w, s], [out0, out1], [
        (cue.Operation([0, 1, 4]), a_), (cue.Operation([0, 2, 4]), b_), (cue.Operation([0, 3, 5]), c_)])
    g = torch.Generator().manual_seed(3)
    Z, R, N = 53, 9, 7
    inputs = [torch.randn(R, x.size, dtype=torch.float64, generator=g).to(dtype),
              torch.randn(R, y.size, dtype=torch.float64, generator=g).to(dtype),
              torch.randn(1, w.size, dtype=torch.float64, generator=g).to(dtype),
              torch.randn(Z, s.size, dtype=torch.float64, generator=g).to(dtype)]
    i0 = torch.randint(0, R, (Z,), generator=g, dtype=torch.int32)
    i1 = torch.randint(0, R, (Z,), generator=g, dtype=torch.int64)
    io = torch.randint(0, N, (Z,), generator=g, dtype=torch.int32)
    check(device, poly, inputs, dtype, input_indices={0: i0, 1: i1}, output_shapes={0: torch.empty(N, 1)}, output_indices={0: io},
          expect_dense=False)


@pytest.mark.gpu
def test_operations_sum_in_the_type_of_the_output(device):
    """Mixed element types: bfloat16 features, float32 weights, the output mapped to the float32 input.  Two operations add
    into that output, one of them reads bfloat16 inputs only: its share must reach the sum in float32 (the reference sums in
    the mapped output type), not rounded to bfloat16 first - a rounding there would show as an error of 2^-9, a hundred
    times the bound of 1e-5 * max|ref| held here (the products of bfloat16 values are formed in float32)."""
    from cuequivariance_amd import cuet

    a_ = random_stp("u,u,u", seed=21)
    b_ = random_stp("u,u,u", seed=22)
    x, y, w, out = a_.operands[0], a_.operands[1], b_.operands[1], a_.operands[2]
    assert b_.operands[0] == x and b_.operands[2] == out
    poly = cue.SegmentedPolynomial([x, y, w], [out], [(cue.Operation([0, 1, 3]), a_), (cue.Operation([0, 2, 3]), b_)])
    g = torch.Generator().manual_seed(4)
    Z = 41
    ins = [torch.randn(Z, x.size, dtype=torch.float64, generator=g).bfloat16(), torch.randn(Z, y.size, dtype=torch.float64, generator=g).bfloat16(),
           torch.randn(Z, w.size, dtype=torch.float64, generator=g).float()]
    m = cuet.SegmentedPolynomial(poly, method="fused_tp", math_dtype=torch.float32, output_dtype_map=[2])
    assert m.m.dense is None
    ref = naive_segmented_polynomial(spec_from_polynomial(poly), [t.double() for t in ins])[0]
    got = m([t.to(device) for t in ins])[0]
    assert got.dtype == torch.float32
    assert rel_err(got, ref) <= 1e-5, rel_err(got, ref)


def test_refusals_match_the_reference():
    from cuequivariance_amd import cuet

    five = STP.from_subscripts("u,u,u,u,u")
    for i in range(5):
        five.add_segment(i, (4,))
    five.add_path(0, 0, 0, 0, 0, c=1.0)
    with pytest.raises(NotImplementedError, match="3 or 4 operands"):
        cuet.SegmentedPolynomial(cue.SegmentedPolynomial.eval_last_operand(five), method="fused_tp", math_dtype=torch.float32)
    empty = STP.from_subscripts("u,u,u")
    for i in range(3):
        empty.add_segment(i, (4,))
    with pytest.raises(NotImplementedError, match="empty paths"):
        cuet.SegmentedPolynomial(cue.SegmentedPolynomial.eval_last_operand(empty), method="fused_tp", math_dtype=torch.float32)
    ok = random_stp("u,u,u", seed=1)
    with pytest.raises(ValueError, match="math_dtype"):
        cuet.SegmentedPolynomial(cue.SegmentedPolynomial.eval_last_operand(ok), method="fused_tp", math_dtype=torch.bfloat16)
