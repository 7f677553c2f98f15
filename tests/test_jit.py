"""Kernels generated, compiled and loaded at first use for a channel-wise descriptor the library was not built for
(``cuequivariance_amd/jit.py``): registration on the CPU, parity against the oracle and against the table-driven kernels
on the GPU."""

import pytest
import torch

from cuequivariance_amd import cue, jit
from cuequivariance_amd.tables import U1dTables
from oracle.naive import naive_segmented_polynomial, spec_from_polynomial


@pytest.fixture
def jit_on(tmp_path, monkeypatch):
    monkeypatch.setenv("CUEQ_AMD_JIT_CACHE", str(tmp_path))
    jit.enable(True)
    yield
    jit.enable(False)


def test_compile_load_and_register(jit_on):
    """A 24-channel l <= 1 product: not in the build's registry; after ``ensure_specialised`` the library reports
    specialised kernels for the forward tables and for the full backward tables, and a second call finds the cached
    object."""
    e = cue.descriptors.channelwise_tensor_product(cue.Irreps("O3", "24x0e+24x1o"), cue.Irreps("O3", "0e+1o"), ["0e", "1o"])
    t = U1dTables.from_polynomial(e.polynomial.flatten_coefficient_modes().squeeze_modes())
    assert not jit._has_spec(t, 0)
    assert jit.ensure_specialised(t, 0)
    assert jit._has_spec(t, 0) and jit._has_spec(t.backward((True, True, True)), 0)
    assert len(list(jit.cache_dir().glob("*.so"))) == 1
    assert jit.ensure_specialised(t, 0)
    # not a channel-wise product: left to the table-driven kernels
    lin = cue.descriptors.spherical_harmonics(cue.SO3(1), [0, 1, 2]).polynomial.flatten_coefficient_modes().squeeze_modes()
    assert not jit.ensure_specialised(U1dTables.from_polynomial(lin), 0)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_jit_kernels_match_oracle_and_generic(device, dtype, jit_on):
    from cuequivariance_amd import cuet

    i1, i2, filt = cue.Irreps("O3", "40x0e+40x1o+40x2e"), cue.Irreps("O3", "0e+1o+2e"), ["0e", "1o", "2e"]
    g = torch.Generator().manual_seed(41)
    N, Z = 31, 500

    def build():
        return cuet.ChannelWiseTensorProduct(i1, i2, filt, layout=cue.ir_mul, shared_weights=False, internal_weights=False,
                                             device=device, dtype=dtype)

    m = build()
    x1 = torch.randn(N, i1.dim, generator=g, dtype=torch.float64).to(dtype)
    x2 = torch.randn(Z, i2.dim, generator=g, dtype=torch.float64).to(dtype)
    w = torch.randn(Z, m.weight_numel, generator=g, dtype=torch.float64).to(dtype)
    snd = torch.randint(0, N, (Z,), generator=g, dtype=torch.int32)
    rcv = torch.sort(torch.randint(0, N, (Z,), generator=g, dtype=torch.int32))[0]
    cot = torch.randn(N, m.irreps_out.dim, generator=g, dtype=torch.float64).to(dtype)

    def run(mod):
        b = [t.clone().to(device).requires_grad_(True) for t in (w, x1, x2)]
        out = mod(b[1], b[2], b[0], indices_1=snd.to(device), indices_out=rcv.to(device), size_out=N)
        return out, torch.autograd.grad(out, b, cot.to(device))

    out, grads = run(m)
    plan = m.f.m._plan(dtype)
    assert plan.specialised(device), "the plan should have found the kernels compiled at first use"
    a = [t.clone().requires_grad_(True) for t in (w, x1, x2)]
    ref = naive_segmented_polynomial(spec_from_polynomial(m.f._polynomial_orig), a, {1: snd}, {0: N}, {0: rcv})[0]
    ref_grads = torch.autograd.grad(ref, a, cot)
    tol = 1e-12 if dtype == torch.float64 else 1e-5

    def err(x, y):
        return (x.detach().cpu().double() - y.double()).abs().max().item() / max(y.abs().max().item(), 1e-30)

    assert err(out, ref) <= tol
    for q, p in zip(grads, ref_grads):
        assert err(q, p) <= tol


@pytest.mark.gpu
def test_jit_symmetric_contraction_matches_generic(device, jit_on, monkeypatch):
    """A 48-channel symmetric contraction (not in the registry): kernels generated at first use for the forward and the
    three backward table sets; results against the table-driven kernels (``CUEQ_FORCE_GENERIC``), which the oracle
    tests of ``tests/test_symmetric_contraction.py`` pin."""
    from cuequivariance_amd import cuet

    m = cuet.SymmetricContraction(cue.Irreps("O3", "48x0e+48x1o+48x2e"), cue.Irreps("O3", "48x0e+48x1o"), 3, 4, layout=cue.ir_mul,
                                  dtype=torch.float32, device=device)
    gen = torch.Generator(device=device).manual_seed(3)
    Z = 700
    x = torch.randn(Z, m.irreps_in.dim, device=device, generator=gen, requires_grad=True)
    idx = torch.randint(0, 4, (Z,), device=device, generator=gen, dtype=torch.int32)
    cot = torch.randn(Z, m.irreps_out.dim, device=device, generator=gen)

    def step():
        out = m(x, idx)
        return [out] + list(torch.autograd.grad(out, [m.weight, x], cot))

    got = step()
    plan = m.f.m._plan(torch.float32)
    assert plan.specialised(device) and plan.backward_plan((True, True)).specialised(device)
    monkeypatch.setenv("CUEQ_FORCE_GENERIC", "1")
    want = step()
    for name, u, v in zip(("out", "dw", "dx"), got, want):
        assert (u - v).abs().max().item() <= 1e-5 * v.abs().max().item(), name
