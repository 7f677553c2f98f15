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


def check(device, poly, inputs, dtype, input_indices=None, output_shapes=None, output_indices=None, expect_dense=None,
          expect_stages=None):
    from cuequivariance_amd import cuet

    m = cuet.SegmentedPolynomial(poly, method="fused_tp", math_dtype=dtype)
    if expect_dense is not None:
        assert (m.m.dense is not None) == expect_dense
    if expect_stages is not None:
        assert (m.m.composed.kind if m.m.composed is not None else None) == expect_stages
        m.m.stages_from = 0  # (the small shapes of these tests would otherwise take the flattened operation)
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


STAGED = {"u,v,uvw,w": "outer", "u,u,uw,w": "same", "u,v,uv,u": "after", "u,v,uv,v": "after",
          "v,u,uvw,w": "outer", "v,u,uv,u": "after"}


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("shared_row", [None, 0, 1])
@pytest.mark.parametrize("form", sorted(STAGED))
def test_forms_with_a_matrix_shape_run_on_the_matrix_cores_when_the_weights_are_shared(device, form, shared_row, dtype):
    """The weights (the operand with two or three modes) as one row: a Linear map on the matrix-core executor with an
    element-wise stage before or after it, not the flattened uniform-1d kernels - also with the two row operands in the other
    order, and with one of them shared over the batch as well.  Results and all three gradients against the oracle."""
    d = random_stp(form, seed=3 + sum(map(ord, form)), nseg=3)
    poly = cue.SegmentedPolynomial.eval_last_operand(d)
    g = torch.Generator().manual_seed(5)
    Z = 203
    rows = [Z, Z, 1]
    if shared_row is not None:
        rows[shared_row] = 1
    inputs = [torch.randn(r, o.size, dtype=torch.float64, generator=g).to(dtype) for r, o in zip(rows, poly.inputs)]
    check(device, poly, inputs, dtype, expect_dense=False, expect_stages=STAGED[form])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("form", ["u,,uw,w", ",v,vw,w"])
def test_fully_connected_form_without_its_unit_mode_runs_on_the_matrix_core_executor(device, form, dtype):
    """``u__uw_w`` / ``_v_vw_w``: the fully connected contraction with the mode of extent one left out of the subscripts (one
    operand is a scalar per segment).  With the weights as one row the wrapper finds the order of the inputs that the
    matrix-core executor takes; results and gradients against the oracle."""
    d = random_stp(form, seed=5 + sum(map(ord, form)), nseg=3)
    poly = cue.SegmentedPolynomial.eval_last_operand(d)
    g = torch.Generator().manual_seed(12)
    inputs = [torch.randn(r, o.size, dtype=torch.float64, generator=g).to(dtype) for r, o in zip((131, 131, 1), poly.inputs)]
    check(device, poly, inputs, dtype, expect_dense=True)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("dims", [dict(u=8, v=4, w=16), dict(u=5, v=3, w=8), dict(u=16, v=12, w=8), dict(u=16, v=8, w=8)])
@pytest.mark.parametrize("form", ["u,v,uvw,w", "v,u,uvw,w"])
def test_outer_product_kernels_against_their_definition(device, form, dims, dtype):
    """``cueq_outer_rows`` and the two ``cueq_outer_rows_contract`` sums through the C ABI against the same sums written with
    index arithmetic in float64 - both orders of the two indices in P, extents that are and are not multiples of four (the
    vector and the scalar kernels), segments read by several parts.  float64 1e-13, float32 1e-5 of the largest value; bfloat16
    and half on inputs rounded to the type: products and sums are formed in float32 and rounded once, half a unit in the last
    place of the largest value (2^-8, 2^-11)."""
    from cuequivariance_amd.cuet.fused_tp import _MatrixWithElementwiseStage, _contract_launch, _outer_launch

    saved = dict(DIMS)
    DIMS.update(dims)
    try:
        d = random_stp(form, seed=17, nseg=3)
    finally:
        DIMS.clear()
        DIMS.update(saved)
    st = _MatrixWithElementwiseStage(cue.SegmentedPolynomial.eval_last_operand(d), torch.float64 if dtype == torch.float64 else torch.float32, "t")
    assert st.kind == "outer" and len(st.parts) > 3
    g = torch.Generator().manual_seed(6)
    Z = 77
    a = torch.randn(Z, st.size[st.i1], dtype=torch.float64, generator=g).to(dtype).double()
    b = torch.randn(Z, st.size[st.i2], dtype=torch.float64, generator=g).to(dtype).double()
    q = torch.randn(Z, st.p_size, dtype=torch.float64, generator=g).to(dtype).double()
    P = torch.zeros(Z, st.p_size, dtype=torch.float64)
    ca, cb = torch.zeros_like(a), torch.zeros_like(b)
    for a_off, b_off, p_off, na, nb in st.parts:
        x, y = a[:, a_off:a_off + na], b[:, b_off:b_off + nb]
        block = x[:, :, None] * y[:, None, :] if st.flag else y[:, :, None] * x[:, None, :]
        P[:, p_off:p_off + na * nb] = block.reshape(Z, -1)
        qb = q[:, p_off:p_off + na * nb].reshape(Z, na, nb) if st.flag else q[:, p_off:p_off + na * nb].reshape(Z, nb, na).transpose(1, 2)
        ca[:, a_off:a_off + na] += (qb * y[:, None, :]).sum(2)
        cb[:, b_off:b_off + nb] += (qb * x[:, :, None]).sum(1)
    tol = {torch.float64: 1e-13, torch.float32: 1e-5, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[dtype]
    ad, bd, qd = (t.to(dtype).to(device) for t in (a, b, q))
    assert rel_err(_outer_launch(st, ad, bd), P) <= tol
    assert rel_err(_contract_launch(st, 0, qd, bd), ca) <= tol
    assert rel_err(_contract_launch(st, 1, qd, ad), cb) <= tol


@pytest.mark.gpu
def test_fully_connected_product_of_general_multiplicities(device):
    """``cuet.FullyConnectedTensorProduct`` with a second operand of multiplicity above one (``uvw,iu,jv,kw`` as it comes from
    the descriptor, mixed multiplicities), float32 and bfloat16, against the oracle in float64 (bfloat16: on the rounded
    inputs, 2e-2): runs as products of the two operands followed by a Linear map.  Rows in ``mul_ir`` against the same
    module in ``ir_mul`` on transposed rows; rows in pieces when the products of all rows exceed the piece size (lowered here)."""
    from cuequivariance_amd import cuet
    from cuequivariance_amd.cuet.fused_tp import _MatrixWithElementwiseStage

    i1, i2, io = cue.Irreps("O3", "32x0e+16x1o"), cue.Irreps("O3", "8x0e+8x1o"), cue.Irreps("O3", "32x0e+32x1o+16x1e")
    e = cue.descriptors.fully_connected_tensor_product(i1, i2, io)
    m = cuet.FullyConnectedTensorProduct(i1, i2, io, layout=cue.ir_mul, shared_weights=True, internal_weights=False, device=device)
    assert isinstance(m.f.m.composed, _MatrixWithElementwiseStage) and m.f.m.composed.kind == "outer"
    g = torch.Generator().manual_seed(8)
    Z = 300
    x1, x2 = torch.randn(Z, i1.dim, generator=g), torch.randn(Z, i2.dim, generator=g)
    w = torch.randn(1, m.weight_numel, generator=g)
    cot = torch.randn(Z, io.dim, generator=g)
    spec = spec_from_polynomial(e.polynomial)
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)):
        b = [t.to(dtype).to(device).requires_grad_(True) for t in (w, x1, x2)]
        a = [t.detach().cpu().double().requires_grad_(True) for t in b]
        ref = naive_segmented_polynomial(spec, a)[0]
        c = cot.to(dtype)
        ref_grads = torch.autograd.grad(ref, a, c.double())
        got = m(b[1], b[2], b[0])
        assert got.dtype == dtype and rel_err(got, ref.detach()) <= tol, (dtype, rel_err(got, ref.detach()))
        grads = torch.autograd.grad(got, b, c.to(device))
        for g_, r_ in zip(grads, ref_grads):
            assert rel_err(g_, r_) <= tol, (dtype, rel_err(g_, r_))
    # mul_ir rows
    mm = cuet.FullyConnectedTensorProduct(i1, i2, io, layout=cue.mul_ir, shared_weights=True, internal_weights=False, device=device)
    to_mul_ir = [cuet.TransposeIrrepsLayout(ir, source=cue.ir_mul, target=cue.mul_ir, device=device) for ir in (i1, i2, io)]
    x1d, x2d, wd = x1.to(device), x2.to(device), w.to(device)
    got = mm(to_mul_ir[0](x1d), to_mul_ir[1](x2d), wd)
    assert rel_err(got, to_mul_ir[2](m(x1d, x2d, wd)).cpu()) <= 1e-6
    # traced as a whole: the stages are torch code around the opaque operators of the matrix-core executor
    compiled = torch.compile(m, fullgraph=True)
    xg = [t.clone().requires_grad_(True) for t in (x1d, x2d, wd)]
    out_c = compiled(xg[0], xg[1], xg[2])
    assert rel_err(out_c, m(x1d, x2d, wd).cpu()) <= 1e-6
    gc = torch.autograd.grad(out_c, xg, cot.to(device))
    xe = [t.clone().requires_grad_(True) for t in (x1d, x2d, wd)]
    ge = torch.autograd.grad(m(xe[0], xe[1], xe[2]), xe, cot.to(device))
    for g_, r_ in zip(gc, ge):
        assert rel_err(g_, r_.cpu()) <= 1e-5
    # no rows at all
    e1, e2 = torch.zeros(0, i1.dim, device=device, requires_grad=True), torch.zeros(0, i2.dim, device=device)
    we = wd.clone().requires_grad_(True)
    empty = m(e1, e2, we)
    assert empty.shape == (0, io.dim)
    assert all(float(g_.abs().sum()) == 0.0 for g_ in torch.autograd.grad(empty.sum(), [e1, we]))
    # rows in pieces
    st = m.f.m.composed
    st.piece_bytes = 64 << 20
    rows = st.piece_bytes // (st.p_size * 4) + 77
    x1d, x2d = torch.randn(rows, i1.dim, device=device), torch.randn(rows, i2.dim, device=device)
    whole = m(x1d, x2d, wd)
    tail = m(x1d[-100:], x2d[-100:], wd)
    assert whole.shape == (rows, io.dim) and rel_err(whole[-100:], tail.cpu()) <= 1e-6
    # products not kept for the backward but formed again there, piece by piece: the same gradients, and second derivatives
    xs = [t.clone().requires_grad_(True) for t in (x1d[:5000], x2d[:5000], wd)]
    ct = torch.randn(5000, io.dim, device=device)

    def grads_and_second(keep):
        st.keep_bytes, st.piece_bytes = keep, 8 << 20
        first = torch.autograd.grad(m(xs[0], xs[1], xs[2]), xs, ct, create_graph=True)
        second = torch.autograd.grad(sum((f * f).sum() for f in first), xs)
        return [f.detach() for f in first] + list(second)

    for kept, again in zip(grads_and_second(32 << 30), grads_and_second(0)):
        assert rel_err(again, kept.cpu()) <= 1e-6


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
