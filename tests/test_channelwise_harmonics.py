"""Channel-wise tensor product with the spherical harmonics of the edge vectors evaluated inside the edge kernels
(``cuet.ChannelWiseSphericalTensorProduct``; the reference runs ``SphericalHarmonics`` - ``cuequivariance_torch/operations/
spherical_harmonics.py:26-93`` - and ``ChannelWiseTensorProduct`` - ``tp_channel_wise.py:30-258`` - one after the other).

Checks: the substituted polynomial against the composition of the two descriptors through the oracle; the module against that
composition (oracle harmonics -> oracle product) for the output and the gradients with respect to weights, node features and
vectors - on the build's unit for the 128-channel l <= 3 descriptor, on the table-driven kernels and on units compiled at first
use."""

import pytest
import torch

from cuequivariance_amd import cue, jit
from cuequivariance_amd.cue import descriptors, fused
from cuequivariance_amd.tables import U1dTables
from oracle.naive import naive_segmented_polynomial, spec_from_polynomial

TOL = {torch.float64: 1e-12, torch.float32: 1e-5}


def composition(irreps1, ls, filt, w, x1, v, snd=None, rcv=None, N=None):
    """Oracle: harmonics of v, then the channel-wise product (gather by snd, scatter-sum by rcv when given)."""
    sh = descriptors.spherical_harmonics(cue.O3(1, -1), ls)
    e = descriptors.channelwise_tensor_product(irreps1, sh.outputs[0].irreps, filt)
    y = naive_segmented_polynomial(spec_from_polynomial(sh.polynomial), [v])[0]
    spec = spec_from_polynomial(e.polynomial)
    if snd is None:
        return naive_segmented_polynomial(spec, [w, x1, y])[0]
    return naive_segmented_polynomial(spec, [w, x1, y], {1: snd}, {0: N}, {0: rcv})[0]


def test_substituted_polynomial_is_the_composition():
    i1 = cue.Irreps("O3", "4x0e+4x1o+4x2e")
    ls, filt = [0, 1, 2, 3], ["0e", "1o", "2e"]
    poly, info, irreps_out = fused.channelwise_spherical(i1, ls, filt)
    assert [len(ope.buffers) for ope, _ in poly.operations] == [3, 4, 5, 6]  # the vector read 0, 1, 2, 3 times
    assert poly.inputs[2].size == 3 and len(info.terms) == 16
    g = torch.Generator().manual_seed(0)
    Z = 9
    v = torch.randn(Z, 3, dtype=torch.float64, generator=g)
    x1 = torch.randn(Z, i1.dim, dtype=torch.float64, generator=g)
    w = torch.randn(Z, poly.inputs[0].size, dtype=torch.float64, generator=g)
    got = naive_segmented_polynomial(spec_from_polynomial(poly), [w, x1, v])[0]
    ref = composition(i1, ls, filt, w, x1, v)
    assert (got - ref).abs().max().item() <= 1e-13 * ref.abs().max().item()
    # the merged terms reproduce the harmonics themselves (Y_1 = sqrt(3) v; sum_m Y_lm^2 = 2l + 1 on unit vectors)
    u = torch.nn.functional.normalize(v, dim=1)
    vals = torch.stack([sum(c * torch.prod(u[:, list(vi)], dim=1) if vi else c * torch.ones(Z, dtype=torch.float64) for vi, c in t)
                        for t in info.terms], dim=1)
    assert torch.allclose(vals[:, 1:4], 3 ** 0.5 * u, atol=1e-14)
    for lo, hi, ell in ((0, 1, 0), (1, 4, 1), (4, 9, 2), (9, 16, 3)):
        assert torch.allclose(vals[:, lo:hi].square().sum(1), torch.full((Z,), 2.0 * ell + 1, dtype=torch.float64), atol=1e-12)


def test_family_detection_and_hashes():
    from cuequivariance_amd import _lib
    import ctypes

    i1 = cue.Irreps("O3", "128x0e+128x1o+128x2e+128x3o")
    poly, info, _ = fused.channelwise_spherical(i1, [0, 1, 2, 3], ["0e", "1o", "2e", "3o"])
    t = U1dTables.from_polynomial(poly)
    assert jit._family(t, poly, info) == "channelwise_sh" and jit.has_fused_backward(t, poly, info)
    assert jit._family(t, poly, None) is None
    lib = _lib.load()
    for tables in (t, t.backward((True, True, True))):  # the build holds the unit for this descriptor
        desc, keep = _lib.make_desc(tables, 0)
        h = ctypes.c_uint64()
        assert lib.cueq_u1d_desc_info(ctypes.byref(desc), ctypes.byref(h)) == 1 and h.value == tables.content_hash(0)


def run_case(device, ir1, ls, filt, N, Z, dtype, seed, normalize=True, layout=cue.ir_mul):
    from cuequivariance_amd import cuet

    i1 = cue.Irreps("O3", ir1)
    m = cuet.ChannelWiseSphericalTensorProduct(i1, ls, filt, normalize=normalize, layout=layout, shared_weights=False,
                                               internal_weights=False, device=device, dtype=dtype)
    g = torch.Generator().manual_seed(seed)
    x1 = torch.randn(N, i1.dim, dtype=torch.float64, generator=g).to(dtype)
    v = torch.randn(Z, 3, dtype=torch.float64, generator=g).to(dtype)
    w = torch.randn(Z, m.weight_numel, dtype=torch.float64, generator=g).to(dtype)
    snd = torch.randint(0, N, (Z,), generator=g, dtype=torch.int32)
    rcv = torch.sort(torch.randint(0, N, (Z,), generator=g, dtype=torch.int32))[0]
    cot = torch.randn(N, m.irreps_out.dim, dtype=torch.float64, generator=g).to(dtype)
    a = [t.double().clone().requires_grad_(True) for t in (w, x1, v)]
    vv = torch.nn.functional.normalize(a[2], dim=1) if normalize else a[2]
    ref = composition(i1, ls, filt, a[0], a[1], vv, snd, rcv, N)
    ref_grads = torch.autograd.grad(ref, a, cot.double())
    b = [t.to(device).requires_grad_(True) for t in (w, x1, v)]
    out = m(b[1], b[2], b[0], indices_1=snd.to(device), indices_out=rcv.to(device), size_out=N)
    grads = torch.autograd.grad(out, b, cot.to(device))
    tol = TOL[dtype]
    for name, got, want in [("out", out, ref), ("dw", grads[0], ref_grads[0]), ("dx1", grads[1], ref_grads[1]), ("dvec", grads[2], ref_grads[2])]:
        err = (got.detach().cpu().double() - want).abs().max().item()
        assert err <= tol * max(want.abs().max().item(), 1e-30), f"{name}: {err:.3e} vs {want.abs().max().item():.3e}"
    return m


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("deterministic", ["0", "1"])
def test_cfg2_descriptor_with_harmonics_in_the_kernels(device, dtype, deterministic, monkeypatch):
    """128 channels, l <= 3, 300 nodes / 4000 edges: the build's unit (forward and the fused backward incl. d/d vectors)."""
    monkeypatch.setenv("CUEQ_DETERMINISTIC", deterministic)
    m = run_case(device, "128x0e+128x1o+128x2e+128x3o", [0, 1, 2, 3], ["0e", "1o", "2e", "3o"], 300, 4000, dtype, seed=41)
    plan = m.f.m._plan(dtype)
    assert plan.specialised(device) and plan.backward_plan((True, True, True)).specialised(device)


@pytest.mark.gpu
@pytest.mark.parametrize("first_use", [False, True])
def test_other_descriptor_with_harmonics(device, first_use, tmp_path, monkeypatch):
    """48 channels, degrees 0..2, unnormalised vectors: the table-driven kernels run the substituted polynomial as it is; with
    compilation at first use the channel-wise generator makes the unit."""
    was = jit.enabled()
    if first_use:
        monkeypatch.setenv("CUEQ_AMD_JIT_CACHE", str(tmp_path))
    jit.enable(first_use)
    try:
        for dtype in (torch.float64, torch.float32):
            m = run_case(device, "48x0e+48x1o+48x1e", [0, 1, 2], ["0e", "1o", "1e", "2o"], 40, 333, dtype, seed=42, normalize=False)
            assert m.f.m._plan(dtype).specialised(device) == first_use
    finally:
        jit.enable(was)


@pytest.mark.gpu
def test_harmonics_with_mul_ir_rows(device, tmp_path, monkeypatch):
    """x1 and the output in mul_ir and the harmonics in the kernels together (a unit compiled at first use)."""
    from cuequivariance_amd import cuet

    def to_mul_ir(x, irreps):  # ir_mul rows -> mul_ir rows by reshapes alone
        outs, off = [], 0
        for mul, ir in irreps:
            outs.append(x[:, off: off + mul * ir.dim].reshape(-1, ir.dim, mul).transpose(1, 2).reshape(x.shape[0], -1))
            off += mul * ir.dim
        return torch.cat(outs, 1)

    monkeypatch.setenv("CUEQ_AMD_JIT_CACHE", str(tmp_path))
    was = jit.enabled()
    jit.enable(True)
    try:
        i1 = cue.Irreps("O3", "32x0e+32x1o+32x2e")
        ls, filt = [0, 1, 2], ["0e", "1o", "2e"]
        a = cuet.ChannelWiseSphericalTensorProduct(i1, ls, filt, layout=cue.ir_mul, shared_weights=False, device=device, dtype=torch.float64)
        b = cuet.ChannelWiseSphericalTensorProduct(i1, ls, filt, layout=cue.mul_ir, shared_weights=False, device=device, dtype=torch.float64)
        g = torch.Generator().manual_seed(43)
        Z = 200
        x1 = torch.randn(Z, i1.dim, dtype=torch.float64, generator=g)
        v = torch.randn(Z, 3, dtype=torch.float64, generator=g).to(device)
        w = torch.randn(Z, a.weight_numel, dtype=torch.float64, generator=g).to(device)
        ya = a(x1.to(device), v, w)
        yb = b(to_mul_ir(x1, i1).to(device), v, w)
        assert (to_mul_ir(ya.cpu(), a.irreps_out) - yb.cpu()).abs().max().item() <= 1e-12 * ya.abs().max().item()
        assert b.f.m._plan(torch.float64).specialised(device)
    finally:
        jit.enable(was)


@pytest.mark.gpu
def test_harmonics_without_edges(device):
    from cuequivariance_amd import cuet

    i1 = cue.Irreps("O3", "128x0e+128x1o+128x2e+128x3o")
    m = cuet.ChannelWiseSphericalTensorProduct(i1, [0, 1, 2, 3], ["0e", "1o", "2e", "3o"], layout=cue.ir_mul, shared_weights=False,
                                               device=device, dtype=torch.float32)
    x1 = torch.randn(6, i1.dim, device=device, requires_grad=True)
    v = torch.randn(0, 3, device=device, requires_grad=True)
    w = torch.randn(0, m.weight_numel, device=device, requires_grad=True)
    idx = torch.zeros(0, dtype=torch.int32, device=device)
    out = m(x1, v, w, indices_1=idx, indices_out=idx, size_out=6)
    assert out.shape == (6, m.irreps_out.dim) and float(out.detach().abs().sum()) == 0.0
    g1, gv, gw = torch.autograd.grad(out, [x1, v, w], torch.ones_like(out))
    assert g1.shape == x1.shape and float(g1.abs().sum()) == 0.0 and gv.shape == (0, 3) and gw.shape == w.shape
