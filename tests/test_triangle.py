"""Triangle multiplicative update: oracle pinning (CPU) and parity of the HIP path (GPU).

The reference's torch entry point forwards to a closed kernel and its own test checks shapes only
(``cuequivariance_torch/tests/primitives/triangle_test.py:97-118``); the algorithm is the open one in
``cuequivariance_jax/cuequivariance_jax/triangle/_triangle_multiplicative_update.py:371-417``.  The oracle restates it
with torch; here it is pinned against library routines (``F.layer_norm``, ``F.linear``) and an explicit loop for the
triangular contraction.  GPU tolerances: float32 ``1e-5 * max|ref|``, bfloat16 ``2e-2 * max|ref|``, float16
``4e-3 * max|ref|`` (intermediates are stored in the input type: a few roundings to 8 / 11 bits each; a kernel that read
half as bfloat16 or the reverse would be off by orders of magnitude) against the float64 oracle evaluated on the inputs
rounded to the tested dtype.
"""

import pytest
import torch
import torch.nn.functional as F

from oracle.triangle import triangle_multiplicative_update as oracle_trimul
from cuequivariance_amd import _lib

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 4e-3}


def make_case(Bsz, N, D, dtype, seed, bias=True, Do=None):
    g = torch.Generator().manual_seed(seed)
    Do = Do or D

    def r(*s):
        return torch.randn(*s, generator=g, dtype=torch.float64)

    p = dict(
        x=r(Bsz, N, N, D), mask=(torch.rand(Bsz, N, N, generator=g) < 0.9).double(),
        norm_in_weight=1 + 0.1 * r(D), norm_in_bias=0.1 * r(D),
        p_in_weight=r(2 * D, D) / D**0.5, g_in_weight=r(2 * D, D) / D**0.5,
        norm_out_weight=1 + 0.1 * r(D), norm_out_bias=0.1 * r(D),
        p_out_weight=r(Do, D) / D**0.5, g_out_weight=r(Do, D) / D**0.5,
    )
    if bias:
        p.update(p_in_bias=0.1 * r(2 * D), g_in_bias=0.1 * r(2 * D), p_out_bias=0.1 * r(Do), g_out_bias=0.1 * r(Do))
    cot = r(Bsz, N, N, Do)
    return {k: v.to(dtype).double() for k, v in p.items()}, cot.to(dtype).double()


@pytest.mark.parametrize("direction", ["outgoing", "incoming"])
def test_oracle_against_library_routines(direction):
    p, _ = make_case(2, 5, 32, torch.float64, 0)
    D = 32
    got = oracle_trimul(direction=direction, **p)
    xh = F.layer_norm(p["x"], (D,), p["norm_in_weight"], p["norm_in_bias"], 1e-5)
    ab = torch.sigmoid(F.linear(xh, p["g_in_weight"], p["g_in_bias"])) * F.linear(xh, p["p_in_weight"], p["p_in_bias"])
    ab = ab * p["mask"].unsqueeze(-1)
    a, b = ab[..., :D], ab[..., D:]
    t = torch.zeros(2, 5, 5, D, dtype=torch.float64)
    for i in range(5):
        for j in range(5):
            for k in range(5):
                if direction == "outgoing":
                    t[:, i, j] += a[:, i, k] * b[:, j, k]
                else:
                    t[:, i, j] += a[:, k, i] * b[:, k, j]
    y = F.layer_norm(t, (D,), p["norm_out_weight"], p["norm_out_bias"], 1e-5)
    want = torch.sigmoid(F.linear(xh, p["g_out_weight"], p["g_out_bias"])) * F.linear(y, p["p_out_weight"], p["p_out_bias"])
    torch.testing.assert_close(got, want, atol=1e-12, rtol=1e-12)


def test_oracle_mask_zeroes_contributions():
    """A fully masked row of the pair tensor contributes nothing to the contraction (outgoing: t[i, j] sums over k)."""
    p, _ = make_case(1, 4, 32, torch.float64, 1, bias=False)
    p["mask"][:] = 1
    full = oracle_trimul(**p)
    p["mask"][0, :, 3] = 0  # drop k = 3 from every sum
    q = {k: v.clone() for k, v in p.items()}
    q["x"] = p["x"].clone()
    dropped = oracle_trimul(**q)
    assert not torch.allclose(full, dropped)
    # changing x at masked positions must leave the projected a, b (hence t) unchanged there, the gate still sees x
    q["mask"][:] = 0
    zero = oracle_trimul(**q)
    # with everything masked t == 0, y == norm_out_bias, so the output is gate * (P_out bias-only projection)
    xh = F.layer_norm(q["x"], (32,), q["norm_in_weight"], q["norm_in_bias"], 1e-5)
    want = torch.sigmoid(xh @ q["g_out_weight"].T) * (q["norm_out_bias"] @ q["p_out_weight"].T)
    torch.testing.assert_close(zero, want, atol=1e-12, rtol=1e-12)


def rel_err(got, ref):
    return (got.double().cpu() - ref).abs().max().item() / max(ref.abs().max().item(), 1e-30)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("direction", ["outgoing", "incoming"])
@pytest.mark.parametrize("shape", [(1, 32, 32, None), (2, 48, 64, None), (1, 40, 128, 64), (1, 33, 32, None), (1, 20, 64, None),
                                   (1, 66, 96, None)])
def test_hip_path_matches_oracle(device, dtype, direction, shape):
    from cuequivariance_amd import cuet

    Bsz, N, D, Do = shape
    p, cot = make_case(Bsz, N, D, dtype, 1, Do=Do)
    pr = {k: v.clone().requires_grad_(k != "mask") for k, v in p.items()}
    ref = oracle_trimul(direction=direction, **pr)
    names = [k for k in pr if k != "mask"]
    ref_grads = torch.autograd.grad(ref, [pr[k] for k in names], cot)
    pg = {k: v.to(dtype).to(device).requires_grad_(k != "mask") for k, v in p.items()}
    out = cuet.triangle_multiplicative_update(direction=direction, **pg)
    assert out.dtype == dtype and out.shape == ref.shape
    grads = torch.autograd.grad(out, [pg[k] for k in names], cot.to(dtype).to(device))
    tol = TOL[dtype]
    assert rel_err(out, ref) <= tol, ("out", rel_err(out, ref))
    for k, got, want in zip(names, grads, ref_grads):
        assert got.dtype == dtype and got.shape == want.shape
        assert rel_err(got, want) <= tol, (k, rel_err(got, want))


@pytest.mark.gpu
@pytest.mark.parametrize("need_affine", [False, True])
@pytest.mark.parametrize("D,M", [(128, 64), (128, 72), (64, 8), (128, 8 * 1001), (64, 64 * 2048 * 2 + 64 * 700 + 24), (128, 64 * 2048 * 3 + 8),
                                 (96, 4104)])
def test_layer_norm_with_layout_change_against_torch(device, D, M, need_affine):
    """``cueq_layer_norm_t_fwd / _bwd`` in bfloat16 on their own (the kernels with one lane per column pair for D = 64 / 128 and
    the tile kernel for other D and for the affine gradients): ragged last tiles, one to three tiles per wavefront, against
    ``F.layer_norm`` in float64 on the same bfloat16 values.  Tolerance 2^-7 of ``max|ref|`` (one rounding of the result)."""
    from cuequivariance_amd.cuet import triangle as tri

    g = torch.Generator(device=device).manual_seed(D + M)
    xt = (torch.randn(D, M, device=device, generator=g) * 1.7 + 0.3).bfloat16()
    gamma = (torch.randn(D, device=device, generator=g) * 0.5 + 1.0).bfloat16()
    beta = torch.randn(D, device=device, generator=g).bfloat16()
    dy = torch.randn(M, D, device=device, generator=g).bfloat16()
    y, mean, rstd = tri.layer_norm_t_fwd(xt, gamma, beta, 1e-5)
    dxt, dgamma, dbeta = tri.layer_norm_t_bwd(dy, xt, mean, rstd, gamma, need_affine)
    x64 = xt.double().t().contiguous().requires_grad_(True)
    g64, b64 = gamma.double().requires_grad_(True), beta.double().requires_grad_(True)
    ref = F.layer_norm(x64, (D,), g64, b64, 1e-5)
    rx, rg, rb = torch.autograd.grad(ref, [x64, g64, b64], dy.double())
    tol = 2.0 ** -7
    assert (y.double() - ref).abs().max().item() <= tol * ref.abs().max().item()
    assert (mean.double() - x64.mean(1)).abs().max().item() <= 1e-5
    assert (dxt.double().t() - rx).abs().max().item() <= tol * rx.abs().max().item()
    if need_affine:
        assert (dgamma.double() - rg).abs().max().item() <= 1e-3 * rg.abs().max().item()
        assert (dbeta.double() - rb).abs().max().item() <= 1e-3 * rb.abs().max().item()


@pytest.mark.gpu
@pytest.mark.parametrize("affine,bias,masked", [(True, True, True), (False, False, False), (True, False, True)])
@pytest.mark.parametrize("M,K,C", [(4096, 128, 256), (4098, 64, 64), (5000, 96, 96), (8192 + 70, 32, 32), (262144, 128, 256)])
def test_layer_norm_fused_into_the_gated_projection(device, M, K, C, affine, bias, masked):
    """``cueq_ln_dual_gate`` (bfloat16): the normalised rows, their statistics and the gated projection against ``F.layer_norm``
    + the two products in float64 on the same bfloat16 values, and against the two separate launches it replaces.  Row counts
    that end inside a 64-row tile, every K the kernel takes, with and without affine weights, biases and mask.  Tolerances
    relative to ``max|ref|``: 2^-7 for the normalised rows (one rounding), 2^-6 for the projection (computed from the rounded
    rows)."""
    from cuequivariance_amd.cuet import triangle as tri

    g = torch.Generator(device=device).manual_seed(M + K + C)
    rn = lambda *shape: torch.randn(*shape, device=device, generator=g)
    x = (rn(M, K) * 1.3 + 0.2).bfloat16()
    gamma = (rn(K) * 0.5 + 1.0).bfloat16() if affine else None
    beta = rn(K).bfloat16() if affine else None
    W1, W2 = (rn(C, K) / K ** 0.5).bfloat16(), (rn(C, K) / K ** 0.5).bfloat16()
    b1, b2 = (rn(C).bfloat16(), rn(C).bfloat16()) if bias else (None, None)
    mask = (torch.rand(M, device=device, generator=g) < 0.8).bfloat16() if masked else None
    fused = tri.ln_dual_gate_fwd(x, gamma, beta, 1e-5, W1, W2, b1, b2, mask)
    assert fused is not None
    out, xh, mean, rstd = fused
    # float64 on the same values; the products take the rounded rows, as the kernels do
    x64 = x.double()
    ref_xh = F.layer_norm(x64, (K,), None if gamma is None else gamma.double(), None if beta is None else beta.double(), 1e-5)
    assert (xh.double() - ref_xh).abs().max().item() <= 2.0 ** -7 * ref_xh.abs().max().item()
    assert (mean.double() - x64.mean(1)).abs().max().item() <= 1e-5
    assert (rstd.double() * torch.sqrt(x64.var(1, unbiased=False) + 1e-5) - 1).abs().max().item() <= 1e-5
    u = xh.double() @ W1.double().t() + (0 if b1 is None else b1.double())
    v = xh.double() @ W2.double().t() + (0 if b2 is None else b2.double())
    ref = torch.sigmoid(u) * v * (1 if mask is None else mask.double()[:, None])
    assert (out.double().t() - ref).abs().max().item() <= 2.0 ** -6 * ref.abs().max().item()
    # the two launches it replaces: for the row lengths that the row kernel sums as a tree of 8-element groups (32, 64, 128) the
    # fused kernel forms its sums in the same order and every bit agrees - a batch that takes the fused launch and a small one
    # that does not give the same rows; for 96 the orders differ
    xh2, mean2, rstd2 = tri.layer_norm_fwd(x, gamma, beta, 1e-5)
    out2 = tri.dual_gate_fwd(W1, W2, xh2, None, b1, b2, 0, mask, 1)
    if K != 96:
        assert torch.equal(mean, mean2) and torch.equal(rstd, rstd2) and torch.equal(xh, xh2) and torch.equal(out, out2)
    else:
        assert (mean - mean2).abs().max().item() <= 1e-6 and (rstd / rstd2 - 1).abs().max().item() <= 1e-6
        assert (xh != xh2).float().mean().item() <= 1e-3
        assert (out.float() - out2.float()).abs().max().item() <= 2.0 ** -6 * out2.float().abs().max().item()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("trans_a,trans_b", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("dims", [(3, 256, 128, 192), (2, 136, 200, 72), (1, 33, 47, 21), (160, 512, 256, 96),
                                  (128, 512, 512, 512)])
def test_gemm_operand_orders(device, dtype, trans_a, trans_b, dims):
    """cueq_gemm against torch.matmul in float64 for the four operand orders: tiled MFMA path (aligned extents,
    partial tiles included), the 256 x 256 tiles (both extents multiples of 256 and at least two tiles per compute
    unit: the last case, which is the contraction of the N = 512, D = 128 update and of its two gradients) and the
    element-wise path (odd extents).  The kernel each case ran on is read back from the library's timing labels."""
    from cuequivariance_amd import _lib
    from cuequivariance_amd.cuet import triangle as tri

    batch, M, N, K = dims
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    aligned = all(v % 8 == 0 for v in (M, N, K))
    big = M % 256 == 0 and N % 256 == 0 and (M // 256) * (N // 256) * batch >= 2 * cus
    if dims == (128, 512, 512, 512):
        assert big or cus > 256, "the benchmark's contraction shape must run on the 256 x 256 tiles"
    label = {torch.float32: "gemm_nt_f32", torch.bfloat16: "gemm_nt_bf16", torch.float16: "gemm_nt_f16"}[dtype] + ("_256" if big else "") if aligned else "gemm_nt_simple"
    g = torch.Generator().manual_seed(M * 7 + N)
    A = torch.randn((batch, K, M) if trans_a else (batch, M, K), generator=g).to(dtype)
    B = torch.randn((batch, K, N) if trans_b else (batch, N, K), generator=g).to(dtype)
    A64 = A.double().transpose(1, 2) if trans_a else A.double()
    B64 = B.double() if trans_b else B.double().transpose(1, 2)
    ref = 0.5 * A64 @ B64
    _lib.timing_begin()
    got = tri.gemm_nt(A.to(device), B.to(device), dtype, alpha=0.5, trans_a=trans_a, trans_b=trans_b)
    ran = _lib.timing_end()
    assert list(ran) == [label], (ran, label)
    assert rel_err(got, ref) <= TOL[dtype], rel_err(got, ref)
    prev = torch.randn(batch, M, N, generator=g).to(dtype)
    got2 = tri.gemm_nt(A.to(device), B.to(device), dtype, out=prev.to(device).clone(), accumulate=True, trans_a=trans_a, trans_b=trans_b)
    assert rel_err(got2, 2 * ref + prev.double()) <= TOL[dtype]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(1, 40, 128, None), (1, 33, 96, 64), (1, 16, 160, None)])
def test_input_gradient_only(device, dtype, shape):
    """Only x asks for a gradient (the benchmark's case): the gate gradients then stay in registers (D <= 128) or go
    through the unfused kernels (D = 160)."""
    from cuequivariance_amd import cuet

    Bsz, N, D, Do = shape
    p, cot = make_case(Bsz, N, D, dtype, 5, Do=Do)
    pr = {k: v.clone() for k, v in p.items()}
    pr["x"].requires_grad_(True)
    (want,) = torch.autograd.grad(oracle_trimul(direction="outgoing", **pr), [pr["x"]], cot)
    pg = {k: v.to(dtype).to(device) for k, v in p.items()}
    pg["x"].requires_grad_(True)
    (got,) = torch.autograd.grad(cuet.triangle_multiplicative_update(direction="outgoing", **pg), [pg["x"]], cot.to(dtype).to(device))
    assert rel_err(got, want) <= TOL[dtype], rel_err(got, want)


@pytest.mark.gpu
def test_defaults_shapes_and_errors(device):
    """The reference's own test: no weights given, shapes only (triangle_test.py:97-118); plus argument checks."""
    from cuequivariance_amd import cuet

    x = torch.randn(1, 32, 32, 32, requires_grad=True, device=device)
    mask = torch.ones(1, 32, 32, device=device)
    out = cuet.triangle_multiplicative_update(x=x, direction="outgoing", mask=mask)
    assert out.shape == (1, 32, 32, 32)
    out.backward(torch.randn_like(out))
    assert x.grad.shape == x.shape and torch.isfinite(x.grad).all()
    # several leading batch dimensions, and none
    y = cuet.triangle_multiplicative_update(torch.randn(2, 3, 8, 8, 32, device=device), "incoming")
    assert y.shape == (2, 3, 8, 8, 32)
    with pytest.raises(ValueError):
        cuet.triangle_multiplicative_update(x, direction="sideways")
    with pytest.raises(ValueError):
        cuet.triangle_multiplicative_update(torch.randn(1, 8, 8, 48, device=device))
    with pytest.raises(ValueError):
        cuet.triangle_multiplicative_update(x, p_in_weight=torch.randn(32, 32, device=device))
    with pytest.raises(ValueError):
        cuet.triangle_multiplicative_update(x.detach().cpu())
    assert int(cuet.TriMulPrecision.IEEE) == 3 and int(cuet.TriMulPrecision.NONE) == -1


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_benchmark_size_against_oracle(device, dtype):
    """The benchmarked case itself (one 512 x 512 pair tensor, 128 channels, bfloat16 - and the same in half -, outgoing,
    Bernoulli(0.9) mask): forward and the gradient with respect to the pair tensor against the float64 oracle evaluated on
    the rounded inputs, 2e-2 (bfloat16) / 4e-3 (half) / 1e-5 (float32) * max|ref|.  This is the only size at which the 256 x 256 contraction tiles, the
    LDS-resident gate backward on 262 144 rows and the LayerNorm with layout change run inside the composed update."""
    from cuequivariance_amd import _lib, cuet

    p, cot = make_case(1, 512, 128, dtype, 7)
    pr = {k: v.clone() for k, v in p.items()}
    pr["x"].requires_grad_(True)
    ref = oracle_trimul(direction="outgoing", **pr)
    (want,) = torch.autograd.grad(ref, [pr["x"]], cot)
    ref = ref.detach()
    pg = {k: v.to(dtype).to(device) for k, v in p.items()}
    pg["x"].requires_grad_(True)
    _lib.timing_begin()
    out = cuet.triangle_multiplicative_update(direction="outgoing", **pg)
    (got,) = torch.autograd.grad(out, [pg["x"]], cot.to(dtype).to(device))
    ran = _lib.timing_end()
    if torch.cuda.get_device_properties(device).multi_processor_count <= 256:
        label = {torch.bfloat16: "gemm_nt_bf16_256", torch.float16: "gemm_nt_f16_256", torch.float32: "gemm_nt_f32_256"}[dtype]
        assert ran.get(label, (0, 0))[0] == 3, ran  # the contraction and its two gradients
    if dtype != torch.float32:  # the stages with the weights resident in the local data share serve both 2-byte formats
        assert "ln_dual_gate_fwd" in ran and "gate_bwd_input_ln" in ran, ran
    assert rel_err(out, ref) <= TOL[dtype], ("out", rel_err(out, ref))
    assert rel_err(got, want) <= TOL[dtype], ("dx", rel_err(got, want))


@pytest.mark.gpu
def test_full_size_properties(device):
    """At the benchmark's size (N = 512, D = 128, bf16): masking everything leaves the bias-only projection, and the two
    directions agree after transposing the pair tensor (outgoing on x^T(i<->k) == incoming on x)."""
    from cuequivariance_amd import cuet

    p, _ = make_case(1, 512, 128, torch.bfloat16, 3, bias=False)
    pg = {k: v.to(torch.bfloat16).to(device) for k, v in p.items()}
    out_in = cuet.triangle_multiplicative_update(direction="incoming", **pg)
    q = dict(pg)
    q["x"] = pg["x"].transpose(1, 2).contiguous()
    q["mask"] = pg["mask"].transpose(1, 2).contiguous()
    # incoming: t[i,j] = sum_k a[k,i] b[k,j]; on the transposed pair tensor the outgoing contraction computes the same t,
    # but the output gate reads x at (i, j) -> compare through zeroed gate weights: sigmoid(0) = 1/2 for both
    pg0, q0 = dict(pg), dict(q)
    pg0["g_out_weight"] = torch.zeros_like(pg["g_out_weight"])
    q0["g_out_weight"] = torch.zeros_like(pg["g_out_weight"])
    a = cuet.triangle_multiplicative_update(direction="incoming", **pg0)
    b = cuet.triangle_multiplicative_update(direction="outgoing", **q0)
    scale = a.float().abs().max().item()
    assert (a.float() - b.float()).abs().max().item() <= 2e-2 * scale
    assert torch.isfinite(out_in.float()).all()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("split", [False, True])
@pytest.mark.parametrize("M", [2048 * 32 + 37 * 32 + 8, 3 * 32 + 8])
def test_gate_bwd_input_many_tiles(device, dtype, split, M):
    """The fused gate backward on more row tiles than one launch holds wavefronts for (each wavefront then walks several
    tiles, the last one partial), against the closed form d/dX of sum(dC * sigmoid(U) * V * mask) written with torch in
    float64: U = W1 X1^T + b1, V = W2 X2^T + b2."""
    from cuequivariance_amd.cuet import triangle as T

    g = torch.Generator().manual_seed(11)
    C, K = 64, 64
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    W1, W2, b1, b2 = r(C, K) / 8, r(C, K) / 8, r(C), r(C)
    X1, X2 = r(M, K), (r(M, K) if split else None)
    mask = (torch.rand(M, generator=g) > 0.2).double()
    dC = r(C, M) if not split else r(M, C)
    prior = r(M, K) if not split else None
    q = lambda t: None if t is None else t.to(dtype)  # the kernel's inputs, rounded once
    W1, W2, b1, b2, X1, X2, mask, dC, prior = map(q, (W1, W2, b1, b2, X1, X2, mask, dC, prior))
    d = lambda t: None if t is None else t.double()
    Xb = d(X2) if split else d(X1)
    U = d(W1) @ d(X1).T + d(b1)[:, None]
    V = d(W2) @ Xb.T + d(b2)[:, None]
    dCm = (d(dC) if not split else d(dC).T) * d(mask)[None, :]
    sg = torch.sigmoid(U)
    dV = dCm * sg
    dU = dCm * V * sg * (1 - sg)
    if split:
        want1, want2 = dU.T @ d(W1), dV.T @ d(W2)
    else:
        want1, want2 = d(prior) + dU.T @ d(W1) + dV.T @ d(W2), None
    dev = lambda t: None if t is None else t.to(device)
    got = T.gate_bwd_input(dev(dC), not split, dev(W1), dev(W2), dev(X1), dev(X2), dev(b1), dev(b2), dev(mask),
                           dX1=dev(prior.clone()) if prior is not None else None, want_gate_grads=True)
    assert got is not None
    g1, g2, gU, gV = got
    tol = TOL[dtype]
    assert rel_err(g1, want1) <= tol, rel_err(g1, want1)
    if split:
        assert rel_err(g2, want2) <= tol, rel_err(g2, want2)
    layout = (lambda t: t) if not split else (lambda t: t.T)
    assert rel_err(gU, layout(dU)) <= tol and rel_err(gV, layout(dV)) <= tol


@pytest.mark.gpu
@pytest.mark.parametrize("with_prior,affine", [(True, True), (False, False), (True, False)])
@pytest.mark.parametrize("M,K,C", [(2048 * 32 + 37 * 32 + 8, 128, 256), (3 * 32 + 8, 64, 64), (1000, 96, 32), (262144, 128, 256)])
def test_gate_bwd_input_through_the_layer_norm(device, M, K, C, with_prior, affine):
    """``cueq_gate_bwd_input_ln`` (bfloat16): the gradient of the input projections continued through the LayerNorm of their
    input, against torch in float64 on the rounded inputs - d/dx of sum(dC * sigmoid(U) * V * mask) + sum(prior * xh) with
    xh = LN(x), U = W1 xh^T + b1, V = W2 xh^T + b2, where xh enters the products as the kernel reads it (rounded to bfloat16)
    and the LayerNorm backward takes the stored mean and 1 / std.  More tiles than wavefronts, a partial last tile, every K."""
    from cuequivariance_amd.cuet import triangle as T

    g = torch.Generator(device=device).manual_seed(M + K + C)
    r = lambda *s: torch.randn(*s, device=device, generator=g)
    x = (r(M, K) * 1.4 + 0.3).bfloat16()
    gamma = (r(K) * 0.5 + 1.0).bfloat16() if affine else None
    beta = r(K).bfloat16() if affine else None
    xh, mean, rstd = T.layer_norm_fwd(x, gamma, beta, 1e-5)
    W1, W2 = (r(C, K) / K ** 0.5).bfloat16(), (r(C, K) / K ** 0.5).bfloat16()
    b1, b2 = r(C).bfloat16(), r(C).bfloat16()
    mask = (torch.rand(M, device=device, generator=g) > 0.2).bfloat16()
    dC = r(C, M).bfloat16()
    prior = r(M, K).bfloat16() if with_prior else None
    got = T.gate_bwd_input_ln(dC, W1, W2, xh, b1, b2, mask, None if prior is None else prior.clone(), x, mean, rstd, gamma)
    assert got is not None and got.shape == (M, K) and got.dtype == torch.bfloat16
    d = lambda t: t.double()
    U = d(W1) @ d(xh).T + d(b1)[:, None]
    V = d(W2) @ d(xh).T + d(b2)[:, None]
    dCm = d(dC) * d(mask)[None, :]
    sg = torch.sigmoid(U)
    dxh = (dCm * V * sg * (1 - sg)).T @ d(W1) + (dCm * sg).T @ d(W2) + (d(prior) if with_prior else 0)
    gg = dxh * (d(gamma) if affine else 1)
    xn = (d(x) - d(mean)[:, None]) * d(rstd)[:, None]
    want = d(rstd)[:, None] * (gg - gg.mean(1, keepdim=True) - xn * (gg * xn).mean(1, keepdim=True))
    assert rel_err(got, want.cpu()) <= TOL[torch.bfloat16], rel_err(got, want.cpu())
    # the two launches it replaces (they round the gradient of xh to bfloat16 in between)
    two = T.gate_bwd_input(dC, True, W1, W2, xh, None, b1, b2, mask, None if prior is None else prior.clone(), False)[0]
    two = T.layer_norm_bwd(two, x, mean, rstd, gamma, False)[0]
    assert rel_err(two, want.cpu()) <= TOL[torch.bfloat16]
    assert (got.float() - two.float()).abs().max().item() <= 2.0 ** -5 * want.abs().max().item()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("N", [64 * 2048 + 64 * 5 + 2, 4096 + 34])
@pytest.mark.parametrize("with_bias", [True, False])
def test_dual_gate_many_column_tiles(device, dtype, N, with_bias):
    """The fused forward gate with a shared right operand on more 64-column tiles than one launch holds wavefronts for
    (each wavefront then walks several tiles; the last tile is partial), against sigmoid(W1 X^T + b1) (W2 X^T + b2) mask
    written with torch in float64 on the rounded inputs."""
    from cuequivariance_amd.cuet import triangle as T

    g = torch.Generator().manual_seed(17)
    C, K = 96, 64
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    W1, W2, X = (r(C, K) / 8).to(dtype), (r(C, K) / 8).to(dtype), r(N, K).to(dtype)
    b1, b2 = (r(C).to(dtype), r(C).to(dtype)) if with_bias else (None, None)
    mask = (torch.rand(N, generator=g) > 0.2).to(dtype)
    d = lambda t: t.double()
    U = d(W1) @ d(X).T + (d(b1)[:, None] if with_bias else 0)
    V = d(W2) @ d(X).T + (d(b2)[:, None] if with_bias else 0)
    want = torch.sigmoid(U) * V * d(mask)[None, :]
    dev = lambda t: None if t is None else t.to(device)
    got = T.dual_gate_fwd(dev(W1), dev(W2), dev(X), None, dev(b1), dev(b2), 0, dev(mask), 1)
    assert got.shape == (C, N) and got.dtype == dtype
    assert rel_err(got, want) <= TOL[dtype], rel_err(got, want)


@pytest.mark.gpu
@pytest.mark.parametrize("with_bias,masked", [(True, False), (False, True), (True, True)])
@pytest.mark.parametrize("M,K,C", [(4096, 128, 128), (32 * 2048 * 2 + 32 * 9 + 5, 64, 96), (5001, 96, 32), (4100, 32, 256)])
def test_dual_gate_two_inputs_result_by_rows(device, M, K, C, with_bias, masked):
    """The forward gate of the output stage in bfloat16 - two inputs of many rows, the weights on the right, biases by column,
    mask by row: the kernel with the weights resident in the local data share (rows past a multiple of 32, more tiles than
    wavefronts, every K) against torch in float64 on the rounded inputs, and bit for bit against the tiled kernel that the
    same call takes for fewer than 4096 rows."""
    from cuequivariance_amd.cuet import triangle as T

    g = torch.Generator(device=device).manual_seed(M + K + C)
    r = lambda *s: torch.randn(*s, device=device, generator=g)
    X1, X2 = r(M, K).bfloat16(), r(M, K).bfloat16()
    W1, W2 = (r(C, K) / K ** 0.5).bfloat16(), (r(C, K) / K ** 0.5).bfloat16()
    b1, b2 = (r(C).bfloat16(), r(C).bfloat16()) if with_bias else (None, None)
    mask = (torch.rand(M, device=device, generator=g) > 0.2).bfloat16() if masked else None
    lib = _lib.load()
    lib.cueq_timing_begin()
    got = T.dual_gate_fwd(X1, X2, W1, W2, b1, b2, 1, mask, 0)
    torch.cuda.synchronize()
    assert dict(_lib.timing_end()).get("dual_gate_fwd", (0, 0))[0] == 1
    d = lambda t: t.double()
    U = d(X1) @ d(W1).T + (d(b1) if with_bias else 0)
    V = d(X2) @ d(W2).T + (d(b2) if with_bias else 0)
    want = torch.sigmoid(U) * V * (d(mask)[:, None] if masked else 1)
    assert got.shape == (M, C) and rel_err(got, want.cpu()) <= TOL[torch.bfloat16], rel_err(got, want.cpu())
    # the same rows in pieces of fewer than 4096: the tiled kernel
    for r0 in (0, M - 3000):
        part = T.dual_gate_fwd(X1[r0:r0 + 3000], X2[r0:r0 + 3000], W1, W2, b1, b2, 1, None if mask is None else mask[r0:r0 + 3000], 0)
        assert torch.equal(part, got[r0:r0 + 3000])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(513, 16384), (37, 8200), (3000, 700), (70000, 130), (1, 8192), (5, 3)])
def test_sum_rows_paths(device, dtype, shape):
    """Column sums of a (rows, cols) matrix in float32: the single-launch kernel (few rows, many columns), the two-stage
    one (everything else), partial column blocks and single rows; against a float64 sum of the rounded input, and
    bit-identical from run to run."""
    from cuequivariance_amd.cuet import triangle as T

    g = torch.Generator().manual_seed(5)
    x = torch.randn(*shape, generator=g).to(dtype)
    want = x.double().sum(0)
    got = T.sum_rows(x.to(device))
    assert got.dtype == torch.float32 and got.shape == (shape[1],)
    scale = x.double().abs().sum(0).max().item()
    assert (got.cpu().double() - want).abs().max().item() <= 1e-6 * scale
    assert torch.equal(got, T.sum_rows(x.to(device)))
