"""``cuet.Linear`` with ``layout=cue.mul_ir`` (the default layout) on the dense kernels that address such rows as they
lie: no ``segmented_transpose`` launch around the call.

The reference transposes in front of and behind its dense kernel (``cuequivariance_torch/operations/linear.py:153-191``
with ``primitives/transpose.py:83-183``); numerically the module is the oracle's Linear applied to the rows converted by
reshapes.  Tolerances relative to ``max|ref|``: float32 1e-5, bfloat16 2e-2, float16 2e-3 (float64 oracle on the rounded inputs).
"""

import pytest
import torch

from cuequivariance_amd import _lib, cue, cuet
from oracle.naive import naive_segmented_polynomial, spec_from_polynomial

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-3}


def to_ir_mul(x, irreps):
    """Rows in mul_ir -> the same rows in ir_mul (pure reshapes)."""
    out, off = [], 0
    for mul, ir in irreps:
        out.append(x[:, off: off + mul * ir.dim].reshape(-1, mul, ir.dim).transpose(1, 2).reshape(-1, mul * ir.dim))
        off += mul * ir.dim
    return torch.cat(out, 1)


def to_mul_ir(x, irreps):
    out, off = [], 0
    for mul, ir in irreps:
        out.append(x[:, off: off + mul * ir.dim].reshape(-1, ir.dim, mul).transpose(1, 2).reshape(-1, mul * ir.dim))
        off += mul * ir.dim
    return torch.cat(out, 1)


def rel_err(got, ref):
    got, ref = got.detach().cpu().double(), ref.detach().cpu().double()
    assert got.shape == ref.shape
    return (got - ref).abs().max().item() / max(ref.abs().max().item(), 1e-30)


def kernel_names(fn):
    lib = _lib.load()
    lib.cueq_timing_begin()
    out = fn()
    torch.cuda.synchronize()
    return out, dict(_lib.timing_end())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize(
    "irreps_in,irreps_out,Z",
    [
        ("128x0e+128x1o+128x2e", "128x0e+128x1o+128x2e", 1000),
        ("64x0e+128x1o+64x2e+64x3o", "128x0e+64x1o+128x2e+64x3o", 333),  # mixed multiplicities, 7 components, ragged rows
        ("64x1o", "128x1o", 17),
        ("128x0e+64x1e+64x1o", "64x0e+128x1e+128x1o", 4097),
    ],
)
def test_linear_mul_ir_matches_oracle_without_transposition(device, dtype, irreps_in, irreps_out, Z):
    irreps_in, irreps_out = cue.Irreps("O3", irreps_in), cue.Irreps("O3", irreps_out)
    m = cuet.Linear(irreps_in, irreps_out, layout=cue.mul_ir, internal_weights=False, method="fused_tp")
    assert m.f_rows is not None
    g = torch.Generator().manual_seed(Z)
    w = torch.randn(1, m.weight_numel, dtype=torch.float64, generator=g).to(dtype).double()
    x = torch.randn(Z, irreps_in.dim, dtype=torch.float64, generator=g).to(dtype).double()  # mul_ir rows
    cot = torch.randn(Z, irreps_out.dim, dtype=torch.float64, generator=g).to(dtype).double()
    # oracle on ir_mul rows
    spec = spec_from_polynomial(m.f._polynomial_orig)
    a = [w.clone().requires_grad_(True), to_ir_mul(x, irreps_in).clone().requires_grad_(True)]
    ref = naive_segmented_polynomial(spec, a)[0]
    ref_gw, ref_gx = torch.autograd.grad(ref, a, to_ir_mul(cot, irreps_out))
    wd = w.to(dtype).to(device).requires_grad_(True)
    xd = x.to(dtype).to(device).requires_grad_(True)

    def step():
        out = m(xd, wd)
        return (out, *torch.autograd.grad(out, [wd, xd], cot.to(dtype).to(device)))

    (out, gw, gx), names = kernel_names(step)
    assert "segmented_transpose" not in names, names
    assert "linear_rows_mul_ir" in names and "linear_dw_mul_ir" in names, names
    tol = TOL[dtype]
    assert rel_err(out, to_mul_ir(ref, irreps_out)) <= tol
    assert rel_err(gx, to_mul_ir(ref_gx, irreps_in)) <= tol
    assert rel_err(gw, ref_gw) <= tol


def test_linear_mul_ir_agrees_with_the_transposing_path_at_full_size(device):
    """200 000 rows (the benchmark's Linear), bfloat16: the module on ``mul_ir`` rows against the same module on ``ir_mul``
    rows fed the converted inputs - same products, same float32 accumulation order per row for the outputs (bit for bit up
    to one rounding step), weight gradient within float32 summation error."""
    irreps = cue.Irreps("O3", "128x0e+128x1o+128x2e")
    m = cuet.Linear(irreps, irreps, layout=cue.mul_ir, internal_weights=False, method="fused_tp")
    r = cuet.Linear(irreps, irreps, layout=cue.ir_mul, internal_weights=False, method="fused_tp")
    Z = 200_000
    g = torch.Generator(device=device).manual_seed(11)
    w = torch.randn(1, m.weight_numel, device=device, generator=g).to(torch.bfloat16).requires_grad_(True)
    x = torch.randn(Z, irreps.dim, device=device, generator=g).to(torch.bfloat16).requires_grad_(True)
    cot = torch.randn(Z, irreps.dim, device=device, generator=g).to(torch.bfloat16)
    (out, gw, gx), names = kernel_names(lambda: (lambda o: (o, *torch.autograd.grad(o, [w, x], cot)))(m(x, w)))
    assert "segmented_transpose" not in names and "transpose" not in names, names
    x2 = to_ir_mul(x.detach(), irreps).requires_grad_(True)
    o2 = r(x2, w)
    gw2, gx2 = torch.autograd.grad(o2, [w, x2], to_ir_mul(cot, irreps))
    assert rel_err(out, to_mul_ir(o2, irreps)) <= 2.0 ** -7
    assert rel_err(gx, to_mul_ir(gx2, irreps)) <= 2.0 ** -7
    assert rel_err(gw, gw2) <= 2.0 ** -7


def test_linear_mul_ir_second_derivatives(device):
    """Gradient of a function of the input gradient (forces and their training): the mul_ir kernels serve the derivative
    functions of the dense executor as well."""
    irreps_in, irreps_out = cue.Irreps("O3", "64x0e+64x1o"), cue.Irreps("O3", "32x0e+64x1o")
    m = cuet.Linear(irreps_in, irreps_out, layout=cue.mul_ir, internal_weights=False, method="fused_tp")
    Z = 50
    g = torch.Generator().manual_seed(3)
    w = torch.randn(1, m.weight_numel, dtype=torch.float64, generator=g).float().double()
    x = torch.randn(Z, irreps_in.dim, dtype=torch.float64, generator=g).float().double()
    spec = spec_from_polynomial(m.f._polynomial_orig)

    def loss(wt, xt, f):
        out = f(wt, xt)
        (gx,) = torch.autograd.grad(out.pow(2).sum(), xt, create_graph=True)
        return (gx.pow(2).sum() + out.sum())

    a = [w.clone().requires_grad_(True), x.clone().requires_grad_(True)]
    ref = loss(a[0], a[1], lambda wt, xt: to_mul_ir(naive_segmented_polynomial(spec, [wt, to_ir_mul(xt, irreps_in)])[0], irreps_out))
    ref_g = torch.autograd.grad(ref, a)
    b = [w.float().to(device).requires_grad_(True), x.float().to(device).requires_grad_(True)]
    got = loss(b[0], b[1], lambda wt, xt: m(xt, wt))
    got_g = torch.autograd.grad(got, b)
    for gg, rr in zip(got_g, ref_g):
        assert rel_err(gg, rr) <= 2e-5


@pytest.fixture
def kernels_at_first_use():
    from cuequivariance_amd import jit

    on = jit.enabled()
    jit.enable(True)
    yield
    jit.enable(on)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize(
    "irreps_in1,irreps_in2,irreps_out,Z",
    [
        ("64x0e+64x1o", "0e+1o+2e", "64x0e+64x1o", 2500),  # the benchmark's product
        ("32x0e+64x1o", "0e+1o", "64x0e+32x1o", 333),  # mixed multiplicities, ragged rows
        ("32x0e+32x2e", "0e+2e", "64x0e+32x2e", 77),  # blocks of 5 components
    ],
)
def test_fully_connected_mul_ir_matches_oracle_without_transposition(device, kernels_at_first_use, dtype, irreps_in1, irreps_in2, irreps_out, Z):
    """The generated fused kernels take mul_ir rows of the first operand and of the output as they lie
    (reference: transposition passes around the kernel, ``cuequivariance_torch/operations/tp_fully_connected.py:118-150``)."""
    i1, i2, i3 = (cue.Irreps("O3", s) for s in (irreps_in1, irreps_in2, irreps_out))
    m = cuet.FullyConnectedTensorProduct(i1, i2, i3, layout=cue.mul_ir, internal_weights=False)
    assert m.f_rows is not None
    g = torch.Generator().manual_seed(Z)
    w = torch.randn(1, m.weight_numel, dtype=torch.float64, generator=g).to(dtype).double()
    x1 = torch.randn(Z, i1.dim, dtype=torch.float64, generator=g).to(dtype).double()  # mul_ir rows
    x2 = torch.randn(Z, i2.dim, dtype=torch.float64, generator=g).to(dtype).double()
    cot = torch.randn(Z, i3.dim, dtype=torch.float64, generator=g).to(dtype).double()
    spec = spec_from_polynomial(m.f._polynomial_orig)
    a = [t.clone().requires_grad_(True) for t in (w, to_ir_mul(x1, i1), x2)]
    ref = naive_segmented_polynomial(spec, a)[0]
    ref_gw, ref_gx1, ref_gx2 = torch.autograd.grad(ref, a, to_ir_mul(cot, i3))
    b = [t.to(dtype).to(device).requires_grad_(True) for t in (w, x1, x2)]

    def step():
        out = m(b[1], b[2], b[0])
        return (out, *torch.autograd.grad(out, b, cot.to(dtype).to(device)))

    (out, gw, gx1, gx2), names = kernel_names(step)
    assert "segmented_transpose" not in names, names
    tol = TOL[dtype]
    assert rel_err(out, to_mul_ir(ref, i3)) <= tol
    assert rel_err(gx1, to_mul_ir(ref_gx1, i1)) <= tol
    assert rel_err(gx2, ref_gx2) <= tol
    assert rel_err(gw, ref_gw) <= tol
