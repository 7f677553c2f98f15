"""GPU parity tests of the dense (MFMA) executor behind ``method="fused_tp"`` against the CPU oracle.

``Linear`` and ``FullyConnectedTensorProduct`` follow the reference's operation tests
(``cuequivariance_torch/tests/operations/linear_test.py:37-96``,
``cuequivariance_torch/tests/operations/tensor_product_test.py:30-108``): outputs and first
derivatives, several dtypes, shared and batched weights.

Tolerances (max-norm relative to ``max|ref|``): float64 1e-12, float32 1e-5, bfloat16 2e-2, float16 2e-3.  The
float64 oracle is evaluated on the inputs after rounding to the tested dtype.
"""

import pytest
import torch

from cuequivariance_amd import cue
from oracle.naive import naive_segmented_polynomial, spec_from_polynomial

pytestmark = pytest.mark.gpu

TOL = {torch.float64: 1e-12, torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-3}


def rel_err(got, ref):
    got, ref = got.detach().cpu().double(), ref.detach().cpu().double()
    assert got.shape == ref.shape, (got.shape, ref.shape)
    return (got - ref).abs().max().item() / max(ref.abs().max().item(), 1e-30)


def check_against_oracle(device, module, inputs, dtype):
    """inputs: float64 host tensors in the polynomial's operand order (weights first)."""
    rounded = [t.to(dtype).double() for t in inputs]
    spec = spec_from_polynomial(module.f._polynomial_orig)
    a = [t.clone().requires_grad_(True) for t in rounded]
    ref = naive_segmented_polynomial(spec, a)[0]
    cot = torch.randn(ref.shape, dtype=torch.float64, generator=torch.Generator().manual_seed(99)).to(dtype).double()
    ref_grads = torch.autograd.grad(ref, a, cot)
    b = [t.to(dtype).to(device).requires_grad_(True) for t in rounded]
    out = module.f(b)[0]
    assert out.dtype == dtype
    grads = torch.autograd.grad(out, b, cot.to(dtype).to(device))
    tol = TOL[dtype]
    assert rel_err(out, ref) <= tol, ("out", rel_err(out, ref))
    for i, (g, r) in enumerate(zip(grads, ref_grads)):
        assert g.dtype == dtype and g.shape == b[i].shape
        assert rel_err(g, r) <= tol, (f"grad {i}", rel_err(g, r))


def linear_module(irreps_in, irreps_out, **kw):
    from cuequivariance_amd import cuet

    return cuet.Linear(cue.Irreps("O3", irreps_in), cue.Irreps("O3", irreps_out), layout=cue.ir_mul,
                       internal_weights=False, method="fused_tp", **kw)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
@pytest.mark.parametrize(
    "irreps_in,irreps_out,Z",
    [
        ("128x0e+128x1o+128x2e", "128x0e+128x1o+128x2e", 1000),  # MFMA path, K = N = 128
        ("64x0e+32x1o+48x2e", "32x0e+64x1o+16x2e", 333),  # mixed multiplicities, ragged row count
        ("32x0e+32x1o", "64x0e+96x1o", 65),
        ("8x0e+3x1o", "5x0e+7x1o", 17),  # sizes the MFMA tiling does not cover
    ],
)
def test_linear_matches_oracle(device, dtype, irreps_in, irreps_out, Z):
    m = linear_module(irreps_in, irreps_out)
    g = torch.Generator().manual_seed(Z)
    w = torch.randn(1, m.weight_numel, dtype=torch.float64, generator=g)
    x = torch.randn(Z, m.irreps_in.dim, dtype=torch.float64, generator=g)
    check_against_oracle(device, m, [w, x], dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
def test_fully_connected_matches_oracle(device, dtype):
    from cuequivariance_amd import cuet

    m = cuet.FullyConnectedTensorProduct(
        cue.Irreps("O3", "64x0e+64x1o"), cue.Irreps("O3", "0e+1o+2e"), cue.Irreps("O3", "64x0e+64x1o"),
        layout=cue.ir_mul, internal_weights=False,
    )
    g = torch.Generator().manual_seed(5)
    w = torch.randn(1, m.weight_numel, dtype=torch.float64, generator=g)
    x1 = torch.randn(777, 256, dtype=torch.float64, generator=g)
    x2 = torch.randn(777, 9, dtype=torch.float64, generator=g)
    check_against_oracle(device, m, [w, x1, x2], dtype)


@pytest.mark.parametrize("layout", [cue.ir_mul, cue.mul_ir])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_fully_connected_benchmark_size(device, dtype, layout):
    """At the benchmark's size (50 000 rows, 64x0e+64x1o (x) 0e+1o+2e -> 64x0e+64x1o): rows drawn from all over the batch
    (the first, the last and those of the last, partly filled tile among them) against the float64 oracle, outputs and
    gradients of the row operands; the weight gradient and the sums over the whole batch through the identities
    <dy, y> = <dL/dw, w> = <dL/dx1, x1> = <dL/dx2, x2> that a product linear in each operand obeys."""
    from cuequivariance_amd import cuet

    m = cuet.FullyConnectedTensorProduct(
        cue.Irreps("O3", "64x0e+64x1o"), cue.Irreps("O3", "0e+1o+2e"), cue.Irreps("O3", "64x0e+64x1o"),
        layout=layout, internal_weights=False,
    )
    Z = 50_000
    g = torch.Generator().manual_seed(11)
    w = (0.2 * torch.randn(1, m.weight_numel, dtype=torch.float64, generator=g)).to(dtype)
    x1 = torch.randn(Z, 256, dtype=torch.float64, generator=g).to(dtype)
    x2 = torch.randn(Z, 9, dtype=torch.float64, generator=g).to(dtype)
    cot = torch.randn(Z, 256, dtype=torch.float64, generator=g).to(dtype)
    a = [t.to(device).requires_grad_(True) for t in (w, x1, x2)]
    y = m(a[1], a[2], a[0])
    assert y.dtype == dtype and y.shape == (Z, 256)
    gw, g1, g2 = torch.autograd.grad(y, a, cot.to(device))
    rows = torch.cat([torch.arange(0, 40), torch.randint(0, Z, (200,), generator=g), torch.arange(Z - 40, Z)])
    b = [w.double().requires_grad_(True), x1[rows].double().requires_grad_(True), x2[rows].double().requires_grad_(True)]
    spec = spec_from_polynomial(m.f._polynomial_orig)
    if layout == cue.mul_ir:  # the oracle's polynomial is written for ir_mul rows: turn the sampled rows
        def to_ir_mul(t, irreps):
            return torch.cat([t[:, o:o + mul * ir.dim].reshape(-1, mul, ir.dim).transpose(1, 2).reshape(len(t), -1)
                              for o, (mul, ir) in zip(_starts(irreps), irreps)], 1)

        def to_mul_ir(t, irreps):
            return torch.cat([t[:, o:o + mul * ir.dim].reshape(-1, ir.dim, mul).transpose(1, 2).reshape(len(t), -1)
                              for o, (mul, ir) in zip(_starts(irreps), irreps)], 1)
    else:
        to_ir_mul = to_mul_ir = lambda t, irreps: t
    ref = naive_segmented_polynomial(spec, [b[0], to_ir_mul(b[1], m.irreps_in1), b[2]])[0]
    ref_rows = to_mul_ir(ref, m.irreps_out)
    r1, r2 = torch.autograd.grad(ref_rows, b[1:], cot[rows].double())
    tol = TOL[dtype]
    assert rel_err(y[rows.to(device)], ref_rows) <= tol
    assert rel_err(g1[rows.to(device)], r1) <= tol
    assert rel_err(g2[rows.to(device)], r2) <= tol
    lhs = (cot.double().to(device) * y.detach().double()).sum().item()
    scale = (cot.double().to(device) * y.detach().double()).abs().sum().item()
    slack = (3e-6 if dtype == torch.float32 else 2e-3) * scale / Z ** 0.5 * 30
    for grad, operand in zip((gw, g1, g2), a):
        assert abs((grad.double() * operand.detach().double()).sum().item() - lhs) <= slack, (grad.shape, lhs, slack)


@pytest.mark.parametrize("layout", [cue.ir_mul, cue.mul_ir])
def test_fully_connected_input_gradients_in_one_pass_and_apart(device, layout, jit_on):
    """Asked for together, the two input gradients of a float32 product come from one kernel that forms the products g W^T
    once (two wavefronts share the channels of a 32-row tile; the halves of dx2 are added in a fixed order); asked for one
    at a time, each comes from its own kernel (the generated kernels of this product are built with the library; the suite
    runs with them switched off unless asked, hence ``jit_on``).  Both ways against each other (different summation orders: 1e-5), the
    one-pass way twice (the same bits), on a batch that ends inside a tile."""
    from cuequivariance_amd import cuet

    m = cuet.FullyConnectedTensorProduct(
        cue.Irreps("O3", "64x0e+64x1o"), cue.Irreps("O3", "0e+1o+2e"), cue.Irreps("O3", "64x0e+64x1o"),
        layout=layout, internal_weights=False,
    )
    Z = 4_133
    g = torch.Generator().manual_seed(17)
    w = (0.2 * torch.randn(1, m.weight_numel, generator=g)).to(device)
    x1 = torch.randn(Z, 256, generator=g).to(device).requires_grad_(True)
    x2 = torch.randn(Z, 9, generator=g).to(device).requires_grad_(True)
    cot = torch.randn(Z, 256, generator=g).to(device)
    both = torch.autograd.grad(m(x1, x2, w), [x1, x2], cot)
    again = torch.autograd.grad(m(x1, x2, w), [x1, x2], cot)
    only1 = torch.autograd.grad(m(x1, x2, w), [x1], cot)[0]
    only2 = torch.autograd.grad(m(x1, x2, w), [x2], cot)[0]
    assert torch.equal(both[0], again[0]) and torch.equal(both[1], again[1])
    assert rel_err(both[0], only1) <= 1e-5 and rel_err(both[1], only2) <= 1e-5
    dense = next(x for x in m.modules() if type(x).__name__ == "SegmentedPolynomialDense" and x.rows_mul_ir == (layout == cue.mul_ir))
    unit = dense.fused_unit(torch.float32, x1.detach(), cot)
    assert unit is not None, "the generated kernels of the benchmark product are built with the library"
    part = torch.empty(1, 18, device=device)
    out1, out2 = torch.empty(1, 256, device=device), torch.empty(1, 9, device=device)
    status = unit.fcj_dx12(1, w.data_ptr(), cot.data_ptr(), 256, x2.data_ptr(), 9, x1.data_ptr(), 256, out1.data_ptr(), 256,
                           out2.data_ptr(), 9, part.data_ptr(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert status == 0, "the one-pass kernel serves this product (multiplicities of 64)"
    assert rel_err(out1, both[0][:1]) <= 1e-5 and rel_err(out2, both[1][:1]) <= 1e-5


def _starts(irreps):
    out, off = [], 0
    for mul, ir in irreps:
        out.append(off)
        off += mul * ir.dim
    return out


def test_linear_module_call_and_internal_weights(device):
    """The module call path (x, weight) and internal weights give what the functional core gives."""
    from cuequivariance_amd import cuet

    irreps = cue.Irreps("O3", "32x0e+32x1o")
    m = cuet.Linear(irreps, irreps, layout=cue.ir_mul, internal_weights=True, method="fused_tp", device=device)
    x = torch.randn(40, irreps.dim, device=device)
    y = m(x)
    y2 = m.f([m.weight, x])[0]
    assert torch.equal(y, y2)
    with pytest.raises(ValueError):
        m(x, torch.randn(1, m.weight_numel, device=device))


def test_linear_empty_batch(device):
    m = linear_module("32x0e+32x1o", "32x0e+32x1o")
    w = torch.randn(1, m.weight_numel, device=device, requires_grad=True)
    x = torch.zeros(0, m.irreps_in.dim, device=device, requires_grad=True)
    y = m(x, w)
    assert y.shape == (0, m.irreps_out.dim)
    gw, gx = torch.autograd.grad(y, [w, x], torch.zeros_like(y))
    assert gx.shape == x.shape and torch.count_nonzero(gw) == 0


def test_linear_full_size_properties(device):
    """At the benchmark's size (200 000 rows x 128 channels x l<=2): linearity in x and in w, and
    agreement of the weight gradient with the adjoint identity <dy, L_w x> = <dL/dw, w>."""
    m = linear_module("128x0e+128x1o+128x2e", "128x0e+128x1o+128x2e")
    Z = 200_000
    g = torch.Generator(device=device).manual_seed(3)
    w = torch.randn(1, m.weight_numel, device=device, generator=g, requires_grad=True)
    x = torch.randn(Z, 1152, device=device, generator=g, requires_grad=True)
    x2 = torch.randn(Z, 1152, device=device, generator=g)
    y = m(x, w)
    y2 = m(x2, w)
    ysum = m(x + 2 * x2, w)
    scale = y.abs().max().item()
    assert (ysum - (y + 2 * y2)).abs().max().item() <= 2e-5 * scale
    cot = torch.randn(Z, 1152, device=device, generator=g)
    gw, gx = torch.autograd.grad(y, [w, x], cot)
    lhs = (cot.double() * y.detach().double()).sum().item()
    assert abs((gw.double() * w.detach().double()).sum().item() - lhs) <= 1e-4 * abs(lhs) + 1e-3 * scale
    assert abs((gx.double() * x.detach().double()).sum().item() - lhs) <= 1e-4 * abs(lhs) + 1e-3 * scale


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize(
    "irreps,classes,sizes",
    [
        # the reference's own case (segmented_polynomial_test.py:480-486: linear 16x0e+16x1o+16x2e, first input indexed)
        ("16x0e+16x1o+16x2e", 4, [70, 0, 1, 200]),
        # MACE-style per-species Linear: 128 channels, 10 species, ragged class sizes around the 128-row tile
        ("128x0e+128x1o+128x2e", 10, [128, 5, 0, 300, 129, 127, 256, 0, 1, 64]),
    ],
)
def test_indexed_linear_matches_oracle(device, dtype, irreps, classes, sizes):
    """``method="indexed_linear"``: one weight row per class, rows sorted by class (grouped MFMA GEMMs), forward and
    the gradients w.r.t. weights and input against the oracle's gather-then-contract evaluation."""
    from cuequivariance_amd import cuet

    m = cuet.Linear(cue.Irreps("O3", irreps), cue.Irreps("O3", irreps), layout=cue.ir_mul, internal_weights=False,
                    weight_classes=classes, method="indexed_linear")
    Z = sum(sizes)
    g = torch.Generator().manual_seed(Z)
    idx = torch.repeat_interleave(torch.arange(classes), torch.tensor(sizes))
    w = torch.randn(classes, m.weight_numel, dtype=torch.float64, generator=g).to(dtype).double()
    x = torch.randn(Z, m.irreps_in.dim, dtype=torch.float64, generator=g).to(dtype).double()
    spec = spec_from_polynomial(m.f._polynomial_orig)
    a = [w.clone().requires_grad_(True), x.clone().requires_grad_(True)]
    ref = naive_segmented_polynomial(spec, a, input_indices={0: idx})[0]
    cot = torch.randn(ref.shape, dtype=torch.float64, generator=g).to(dtype).double()
    ref_grads = torch.autograd.grad(ref, a, cot)
    wg = w.to(dtype).to(device).requires_grad_(True)
    xg = x.to(dtype).to(device).requires_grad_(True)
    out = m(xg, wg, idx.to(torch.int32).to(device))
    assert out.dtype == dtype and out.shape == ref.shape
    grads = torch.autograd.grad(out, [wg, xg], cot.to(dtype).to(device))
    tol = TOL[dtype]
    assert rel_err(out, ref) <= tol, ("out", rel_err(out, ref))
    for name, got, want in zip(("dw", "dx"), grads, ref_grads):
        assert rel_err(got, want) <= tol, (name, rel_err(got, want))
    # int64 indices give the same bits; unsorted indices are refused like in the reference
    out64 = m(xg, wg, idx.to(device))
    assert torch.equal(out64, out)
    if Z > 2:
        with pytest.raises(AssertionError):
            m(xg, wg, idx.flip(0).to(device))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_weights_per_sample_and_unsorted_classes(device, dtype):
    """``shared_weights=False`` (one weight row per sample) for the fully connected product and the linear map, and
    ``weight_classes`` with an index in arbitrary order: served by the uniform-1d kernels on the flattened descriptor;
    against the CPU oracle on the unflattened descriptor (reference behaviour:
    ``cuequivariance_torch/operations/tp_fully_connected.py:30-207``, ``operations/linear.py:150-190``)."""
    from cuequivariance_amd import cuet

    g = torch.Generator().manual_seed(23)
    Z = 77
    tol = 1e-12 if dtype == torch.float64 else 1e-5
    i1, i2, io = cue.Irreps("O3", "6x0e+4x1o"), cue.Irreps("O3", "0e+1o"), cue.Irreps("O3", "6x0e+4x1o+2x2e")
    fc = cuet.FullyConnectedTensorProduct(i1, i2, io, layout=cue.ir_mul, shared_weights=False, device=device, dtype=dtype)
    x1 = torch.randn(Z, i1.dim, generator=g, dtype=torch.float64).to(dtype)
    x2 = torch.randn(Z, i2.dim, generator=g, dtype=torch.float64).to(dtype)
    w = torch.randn(Z, fc.weight_numel, generator=g, dtype=torch.float64).to(dtype)
    spec = spec_from_polynomial(cue.descriptors.fully_connected_tensor_product(i1, i2, io).polynomial)
    a = [t.clone().requires_grad_(True) for t in (w, x1, x2)]
    ref = naive_segmented_polynomial(spec, a)[0]
    cot = torch.randn(ref.shape, generator=g, dtype=torch.float64).to(dtype)
    ref_grads = torch.autograd.grad(ref, a, cot)
    b = [t.clone().to(device).requires_grad_(True) for t in (w, x1, x2)]
    out = fc(b[1], b[2], b[0])
    grads = torch.autograd.grad(out, b, cot.to(device))
    assert rel_err(out, ref) <= tol, "fc per-sample weights"
    for p, q, name in zip(ref_grads, grads, ("dw", "dx1", "dx2")):
        assert rel_err(q, p) <= tol, name

    lin = cuet.Linear(i1, io, layout=cue.ir_mul, weight_classes=4, device=device, dtype=dtype)
    idx = torch.randint(0, 4, (Z,), generator=g, dtype=torch.int32)  # not sorted
    spec = spec_from_polynomial(cue.descriptors.linear(i1, io).polynomial)
    wl = lin.weight.detach().cpu().clone().requires_grad_(True)
    xl = x1.clone().requires_grad_(True)
    ref = naive_segmented_polynomial(spec, [wl, xl], {0: idx})[0]
    cot = torch.randn(ref.shape, generator=g, dtype=torch.float64).to(dtype)
    ref_grads = torch.autograd.grad(ref, [wl, xl], cot)
    xg = x1.clone().to(device).requires_grad_(True)
    out = lin(xg, weight_indices=idx.to(device))
    grads = torch.autograd.grad(out, [lin.weight, xg], cot.to(device))
    assert rel_err(out, ref) <= tol, "linear with unsorted classes"
    for p, q, name in zip(ref_grads, grads, ("dw", "dx")):
        assert rel_err(q, p) <= tol, name

    lin2 = cuet.Linear(i1, io, layout=cue.ir_mul, shared_weights=False, device=device, dtype=dtype)
    wz = torch.randn(Z, lin2.weight_numel, generator=g, dtype=torch.float64).to(dtype)
    ref = naive_segmented_polynomial(spec, [wz, x1])[0]
    assert rel_err(lin2(x1.to(device), wz.to(device)), ref) <= tol, "linear per-sample weights"


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_linear_second_derivatives_match_oracle(device, dtype):
    """Force training differentiates a gradient again: the gradients of the 3-operand form are functions of their own
    (each differentiable in terms of the other two), so ``create_graph=True`` stays on the MFMA kernels.  Against
    autograd through the CPU oracle, all second derivatives of a scalar built from the input gradient."""
    m = linear_module("32x0e+32x1o+16x2e", "16x0e+32x1o+32x2e")
    g = torch.Generator().manual_seed(11)
    Z = 70
    w = torch.randn(1, m.weight_numel, dtype=torch.float64, generator=g).to(dtype).double()
    x = torch.randn(Z, m.irreps_in.dim, dtype=torch.float64, generator=g).to(dtype).double()
    cot = torch.randn(Z, m.irreps_out.dim, dtype=torch.float64, generator=g).to(dtype).double()
    v = torch.randn(Z, m.irreps_in.dim, dtype=torch.float64, generator=g).to(dtype).double()
    u = torch.randn(1, m.weight_numel, dtype=torch.float64, generator=g).to(dtype).double()
    spec = spec_from_polynomial(m.f._polynomial_orig)

    def second(fwd, w_, x_, dev_, dt):
        out = fwd(w_, x_)
        gw, gx = torch.autograd.grad(out, [w_, x_], cot.to(dt).to(dev_), create_graph=True)
        s = (gx * v.to(dt).to(dev_)).sum() + (gw * u.to(dt).to(dev_)).sum() + (gx * gx).sum()
        return torch.autograd.grad(s, [w_, x_])

    a = [w.clone().requires_grad_(True), x.clone().requires_grad_(True)]
    want = second(lambda w_, x_: naive_segmented_polynomial(spec, [w_, x_])[0], *a, torch.device("cpu"), torch.float64)
    b = [w.to(dtype).to(device).requires_grad_(True), x.to(dtype).to(device).requires_grad_(True)]
    got = second(lambda w_, x_: m.f([w_, x_])[0], *b, device, dtype)
    tol = 1e-12 if dtype == torch.float64 else 2e-5
    for name, p, q in zip(("d/dw", "d/dx"), got, want):
        assert rel_err(p, q) <= tol, (name, rel_err(p, q))


def fc_second_derivatives(device, dtype, irreps, Z=60):
    """All second derivatives of a scalar built from the three first gradients of a fully connected product: GPU module
    against autograd through the CPU oracle.  Returns the largest relative error."""
    from cuequivariance_amd import cuet

    ir = cue.Irreps("O3", irreps)
    m = cuet.FullyConnectedTensorProduct(ir, cue.Irreps("O3", "0e+1o"), ir, layout=cue.ir_mul, internal_weights=False)
    g = torch.Generator().manual_seed(12)
    ins = [torch.randn(1, m.weight_numel, dtype=torch.float64, generator=g), torch.randn(Z, ir.dim, dtype=torch.float64, generator=g),
           torch.randn(Z, 4, dtype=torch.float64, generator=g)]
    ins = [t.to(dtype).double() for t in ins]
    cot = torch.randn(Z, ir.dim, dtype=torch.float64, generator=g).to(dtype).double()
    probes = [torch.randn(t.shape, dtype=torch.float64, generator=g).to(dtype).double() for t in ins]
    spec = spec_from_polynomial(m.f._polynomial_orig)

    def second(fwd, a, dev_, dt):
        out = fwd(a)
        grads = torch.autograd.grad(out, a, cot.to(dt).to(dev_), create_graph=True)
        s = sum((gr * p.to(dt).to(dev_)).sum() for gr, p in zip(grads, probes)) + (grads[1] * grads[1]).sum()
        return torch.autograd.grad(s, a)

    want = second(lambda a: naive_segmented_polynomial(spec, a)[0], [t.clone().requires_grad_(True) for t in ins], torch.device("cpu"), torch.float64)
    got = second(lambda a: m.f(a)[0], [t.to(dtype).to(device).requires_grad_(True) for t in ins], device, dtype)
    return max(rel_err(p, q) for p, q in zip(got, want)), m


def test_fully_connected_second_derivatives_match_oracle(device):
    """The four trilinear forms (product and its three gradients) are closed under differentiation: ``create_graph=True``
    stays on the fully connected kernels (here the table-driven ones; ``tests/test_jit.py`` covers the generated ones)."""
    err, _ = fc_second_derivatives(device, torch.float32, "32x0e+32x1o")
    assert err <= 2e-5, err


def test_fully_connected_float64_second_derivatives_match_oracle(device):
    """float64 runs the per-path kernels; the same closure of four forms makes them differentiable to any order."""
    err, _ = fc_second_derivatives(device, torch.float64, "8x0e+8x1o")
    assert err <= 1e-12, err


@pytest.mark.parametrize("layout", [cue.ir_mul, cue.mul_ir])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_fully_connected_with_scalar_attributes_matches_oracle(device, dtype, layout):
    """A second operand of several invariant scalars (node attributes, ``5x0e``) is outside the 4-operand dense form; the
    module evaluates it as the Linear map of the features ``x1[i, u] x2[v]`` with the same weights.  Forward, gradients
    and second derivatives against the CPU oracle on the fully connected descriptor itself."""
    from cuequivariance_amd import cuet

    i1, i2, i3 = cue.Irreps("O3", "16x0e+16x1o+8x0e"), cue.Irreps("O3", "5x0e"), cue.Irreps("O3", "16x0e+8x1o")
    m = cuet.FullyConnectedTensorProduct(i1, i2, i3, layout=layout, internal_weights=False)
    assert m.f is not None and m.f.m.dense is None and m.f.m.composed.kind == "outer"
    m.f.m.stages_from = 0  # (these small multiplicities would otherwise take the flattened operation)
    g = torch.Generator().manual_seed(13)
    Z = 45
    ins = [torch.randn(1, m.weight_numel, dtype=torch.float64, generator=g), torch.randn(Z, i1.dim, dtype=torch.float64, generator=g),
           torch.randn(Z, i2.dim, dtype=torch.float64, generator=g)]
    ins = [t.to(dtype).double() for t in ins]
    cot = torch.randn(Z, i3.dim, dtype=torch.float64, generator=g).to(dtype).double()
    ref_mod = cuet.FullyConnectedTensorProduct(i1, i2, i3, layout=cue.ir_mul, internal_weights=False)
    spec = spec_from_polynomial(ref_mod.f_per_sample._polynomial)

    def columns(irreps):  # index of every ir_mul column in a row of the tested layout
        idx, off = [], 0
        for mul, ir in irreps:
            d = ir.dim
            idx += [off + (u * d + i if layout == cue.mul_ir else i * mul + u) for i in range(d) for u in range(mul)]
            off += mul * d
        return torch.tensor(idx)

    c1, c2, c3 = columns(i1), columns(i2), columns(i3)

    def oracle(a):  # the oracle works on ir_mul rows; the layout changes are permutations of columns
        out = naive_segmented_polynomial(spec, [a[0], a[1][:, c1], a[2][:, c2]])[0]
        return out[:, torch.argsort(c3)]

    def run(fwd, a, dev_, dt):
        out = fwd(a)
        grads = torch.autograd.grad(out, a, cot.to(dt).to(dev_), create_graph=True)
        second = torch.autograd.grad((grads[1] * grads[1]).sum() + (grads[0] * grads[0]).sum(), a)
        return (out,) + grads + second

    want = run(oracle, [t.clone().requires_grad_(True) for t in ins], torch.device("cpu"), torch.float64)
    got = run(lambda a: m(a[1], a[2], a[0]), [t.to(dtype).to(device).requires_grad_(True) for t in ins], device, dtype)
    tol = 1e-12 if dtype == torch.float64 else 2e-5
    for i, (p, q) in enumerate(zip(got, want)):
        assert rel_err(p, q) <= tol, (i, rel_err(p, q))


def test_indexed_linear_second_derivatives_match_oracle(device):
    """The indexed Linear under ``create_graph=True``: second derivatives against autograd through the oracle's
    gather-then-contract evaluation."""
    from cuequivariance_amd import cuet

    irreps = cue.Irreps("O3", "16x0e+16x1o")
    m = cuet.Linear(irreps, irreps, layout=cue.ir_mul, internal_weights=False, weight_classes=3, method="indexed_linear")
    g = torch.Generator().manual_seed(14)
    Z = 50
    x = torch.randn(Z, irreps.dim, dtype=torch.float64, generator=g).float().double()
    w = torch.randn(3, m.weight_numel, dtype=torch.float64, generator=g).float().double()
    cot = torch.randn(Z, irreps.dim, dtype=torch.float64, generator=g).float().double()
    idx = torch.sort(torch.randint(0, 3, (Z,), generator=g, dtype=torch.int32))[0]
    spec = spec_from_polynomial(m.f._polynomial_orig)

    def second(fwd, a, dev_, dt):
        out = fwd(a)
        gw, gx = torch.autograd.grad(out, a, cot.to(dt).to(dev_), create_graph=True)
        return torch.autograd.grad((gx * gx).sum() + (gw * gw).sum(), a)

    want = second(lambda a: naive_segmented_polynomial(spec, [a[0], a[1]], {0: idx}, {}, {})[0],
                  [w.clone().requires_grad_(True), x.clone().requires_grad_(True)], torch.device("cpu"), torch.float64)
    got = second(lambda a: m(a[1], a[0], weight_indices=idx.to(device)),
                 [w.float().to(device).requires_grad_(True), x.float().to(device).requires_grad_(True)], device, torch.float32)
    for name, p, q in zip(("d/dw", "d/dx"), got, want):
        assert rel_err(p, q) <= 2e-5, (name, rel_err(p, q))
