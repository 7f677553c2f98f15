"""torch.compile(fullgraph=True) of modules on the uniform-1d path: the launch is one opaque operator
(``cuequivariance_amd::u1d_launch``) with a shape function and a registered backward; results must equal eager mode.
The ``aot_eager`` backend is used: it exercises Dynamo and AOT autograd (what ``fullgraph`` is about) without a code
generator for the surrounding element-wise work.  The reference checks the same modes in
``cuequivariance_torch/cuequivariance_torch/_tests/utils.py:128-210``."""

import pytest
import torch

from cuequivariance_amd import cue


@pytest.mark.gpu
@pytest.mark.parametrize("indexed", [False, True])
def test_compiled_channelwise_matches_eager(device, indexed):
    from cuequivariance_amd import cuet

    m = cuet.ChannelWiseTensorProduct(cue.Irreps("O3", "32x0e+32x1o+32x2e"), cue.Irreps("O3", "0e+1o+2e"), ["0e", "1o", "2e"],
                                      layout=cue.ir_mul, shared_weights=False, internal_weights=False, device=device,
                                      dtype=torch.float32)
    g = torch.Generator(device=device).manual_seed(3)
    N, Z = 50, 700
    x1 = torch.randn(N if indexed else Z, m.irreps_in1.dim, device=device, generator=g, requires_grad=True)
    x2 = torch.randn(Z, m.irreps_in2.dim, device=device, generator=g, requires_grad=True)
    w = torch.randn(Z, m.weight_numel, device=device, generator=g, requires_grad=True)
    snd = torch.randint(0, N, (Z,), device=device, generator=g, dtype=torch.int32)
    rcv = torch.sort(torch.randint(0, N, (Z,), device=device, generator=g, dtype=torch.int32))[0]

    def f(x1, x2, w):
        if indexed:
            return m(x1, x2, w, indices_1=snd, indices_out=rcv, size_out=N)
        return m(x1, x2, w)

    ref = f(x1, x2, w)
    cot = torch.randn(ref.shape, device=device, generator=g)
    ref_grads = torch.autograd.grad(ref, [x1, x2, w], cot)
    fc = torch.compile(f, fullgraph=True, backend="aot_eager", dynamic=False)
    for _ in range(2):  # second call: the cached graph
        out = fc(x1, x2, w)
        grads = torch.autograd.grad(out, [x1, x2, w], cot)
        assert torch.equal(out, ref)
        for a, b, name in zip(grads, ref_grads, ("dx1", "dx2", "dw")):
            if indexed and name == "dx1":  # scattered with floating-point atomics: the summation order varies
                torch.testing.assert_close(a, b, rtol=0, atol=1e-5 * float(b.abs().max()))
            else:
                assert torch.equal(a, b), name


@pytest.mark.gpu
def test_compiled_symmetric_contraction_and_harmonics(device):
    from cuequivariance_amd import cuet

    sc = cuet.SymmetricContraction(cue.Irreps("O3", "32x0e+32x1o+32x2e"), cue.Irreps("O3", "32x0e+32x1o"), 3, 5,
                                   layout=cue.ir_mul, dtype=torch.float32, device=device)
    sh = cuet.SphericalHarmonics([0, 1, 2, 3], normalize=True, device=device)
    g = torch.Generator(device=device).manual_seed(1)
    x = torch.randn(300, sc.irreps_in.dim, device=device, generator=g, requires_grad=True)
    idx = torch.randint(0, 5, (300,), device=device, generator=g, dtype=torch.int32)
    v = torch.randn(300, 3, device=device, generator=g, requires_grad=True)

    def f(x, v):
        return sc(x, idx).sum(dim=1, keepdim=True) * sh(v)

    ref = f(x, v)
    cot = torch.randn(ref.shape, device=device, generator=g)
    ref_grads = torch.autograd.grad(ref, [x, v, sc.weight], cot)
    fc = torch.compile(f, fullgraph=True, backend="aot_eager", dynamic=False)
    out = fc(x, v)
    grads = torch.autograd.grad(out, [x, v, sc.weight], cot)
    torch.testing.assert_close(out, ref, rtol=1e-6, atol=1e-6 * float(ref.detach().abs().max()))
    for a, b in zip(grads, ref_grads):
        torch.testing.assert_close(a, b, rtol=1e-6, atol=1e-5 * float(b.abs().max()))


@pytest.mark.gpu
def test_export_channelwise(device):
    """``torch.export.export`` of the module: one ``u1d_launch`` node, the exported program reproduces eager mode."""
    from cuequivariance_amd import cuet

    m = cuet.ChannelWiseTensorProduct(cue.Irreps("O3", "32x0e+32x1o"), cue.Irreps("O3", "0e+1o"), ["0e", "1o"],
                                      layout=cue.ir_mul, shared_weights=False, internal_weights=False, device=device,
                                      dtype=torch.float32)
    g = torch.Generator(device=device).manual_seed(8)
    x1 = torch.randn(100, m.irreps_in1.dim, device=device, generator=g)
    x2 = torch.randn(100, m.irreps_in2.dim, device=device, generator=g)
    w = torch.randn(100, m.weight_numel, device=device, generator=g)
    ep = torch.export.export(m, (x1, x2, w))
    targets = [str(n.target) for n in ep.graph.nodes if n.op == "call_function"]
    assert any("u1d_launch" in t for t in targets)
    assert torch.equal(ep.module()(x1, x2, w), m(x1, x2, w))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_compiled_triangle_update_matches_eager(device, dtype):
    """``triangle_multiplicative_update`` under ``torch.compile(fullgraph=True)``: forward and backward are the opaque
    operators ``trimul_fwd`` / ``trimul_bwd`` around the same launches, so results are bit-identical to eager mode."""
    from cuequivariance_amd import cuet

    g = torch.Generator(device=device).manual_seed(12)
    D, N = 64, 24
    r = lambda *s: torch.randn(*s, device=device, generator=g).to(dtype)
    x = r(2, N, N, D).requires_grad_(True)
    mask = (torch.rand(2, N, N, device=device, generator=g) > 0.2).to(dtype)
    w = dict(p_in_weight=(r(2 * D, D) / 8).requires_grad_(True), g_in_weight=(r(2 * D, D) / 8).requires_grad_(True),
             p_out_weight=(r(D, D) / 8).requires_grad_(True), g_out_weight=(r(D, D) / 8).requires_grad_(True),
             norm_in_weight=(1 + 0.1 * r(D)).requires_grad_(True), g_in_bias=(0.1 * r(2 * D)).requires_grad_(True))

    def f(x, mask, w):
        return cuet.triangle_multiplicative_update(x, direction="incoming", mask=mask, **w)

    ref = f(x, mask, w)
    cot = r(*ref.shape)
    leaves = [x, *w.values()]
    ref_grads = torch.autograd.grad(ref, leaves, cot)
    out = torch.compile(f, fullgraph=True, backend="aot_eager", dynamic=False)(x, mask, w)
    assert torch.equal(out, ref)
    for a, b in zip(torch.autograd.grad(out, leaves, cot), ref_grads):
        assert a.dtype == b.dtype and torch.equal(a, b)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_compiled_linear_and_fully_connected_match_eager(device, dtype):
    """The MFMA executor (shared weights) under ``torch.compile(fullgraph=True)``: ``dense_fwd`` / ``dense_bwd``."""
    from cuequivariance_amd import cuet

    g = torch.Generator(device=device).manual_seed(21)
    i1, i2, io = cue.Irreps("O3", "64x0e+64x1o"), cue.Irreps("O3", "0e+1o+2e"), cue.Irreps("O3", "64x0e+64x1o")
    lin = cuet.Linear(i1, io, layout=cue.ir_mul, device=device, dtype=dtype)
    fc = cuet.FullyConnectedTensorProduct(i1, i2, io, layout=cue.ir_mul, device=device, dtype=dtype)
    x1 = torch.randn(300, i1.dim, device=device, generator=g).to(dtype).requires_grad_(True)
    x2 = torch.randn(300, i2.dim, device=device, generator=g).to(dtype).requires_grad_(True)

    def f(x1, x2):
        return fc(lin(x1), x2)

    ref = f(x1, x2)
    cot = torch.randn(ref.shape, device=device, generator=g).to(dtype)
    leaves = [x1, x2, lin.weight, fc.weight]
    ref_grads = torch.autograd.grad(ref, leaves, cot)
    out = torch.compile(f, fullgraph=True, backend="aot_eager", dynamic=False)(x1, x2)
    assert torch.equal(out, ref)
    for a, b in zip(torch.autograd.grad(out, leaves, cot), ref_grads):
        assert torch.equal(a, b)
