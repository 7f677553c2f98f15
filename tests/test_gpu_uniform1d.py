"""GPU parity tests of the uniform-1d executor (through the C ABI) against the CPU oracle.

Tolerances (max-norm): float64 ``|err| <= 1e-12 * max|ref|``; float32 ``<= 1e-5 * max|ref|``;
bfloat16 / float16 ``<= 2e-2 * max|ref|``.  Integer outputs (CSR grouping) are compared exactly.

Cases follow the reference's own test matrix: every combination of shared / batched / indexed
operands (``cuequivariance_torch/tests/primitives/segmented_polynomial_test.py:286-301``), several
dtype / math dtype pairs (``:270-280``), first and second derivatives (``:148-171``), gather/scatter
equivalence (``cuequivariance_torch/tests/operations/channel_wise_test.py:231-305``), plus empty and
ragged inputs.
"""

import itertools
import os

import pytest
import torch

from cuequivariance_amd import cue
from cuequivariance_amd.tables import U1dTables
from oracle.naive import naive_segmented_polynomial, spec_from_polynomial

pytestmark = pytest.mark.gpu

TOL = {torch.float64: 1e-12, torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-2}


def assert_close(got: torch.Tensor, ref: torch.Tensor, tol: float, what: str = ""):
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    got, ref = got.detach().cpu().double(), ref.detach().cpu().double()
    scale = max(ref.abs().max().item(), 1e-30) if ref.numel() else 1.0
    err = (got - ref).abs().max().item() if ref.numel() else 0.0
    assert err <= tol * scale, f"{what}: max err {err:.3e} > {tol:.0e} * {scale:.3e}"


def cw_module(irreps1, irreps2, filt, **kw):
    from cuequivariance_amd import cuet

    return cuet.ChannelWiseTensorProduct(
        cue.Irreps("O3", irreps1), cue.Irreps("O3", irreps2), filt, layout=cue.ir_mul, shared_weights=False, **kw
    )


def run_cw_case(device, m, N, Z, dtype, seed, sort_receivers=True, index_dtype=torch.int32, tol=None):
    spec = spec_from_polynomial(m.f._polynomial_orig)
    g = torch.Generator().manual_seed(seed)
    D1, D2, W, D3 = m.irreps_in1.dim, m.irreps_in2.dim, m.weight_numel, m.irreps_out.dim
    x1 = torch.randn(N, D1, dtype=torch.float64, generator=g).to(dtype)
    x2 = torch.randn(Z, D2, dtype=torch.float64, generator=g).to(dtype)
    w = torch.randn(Z, W, dtype=torch.float64, generator=g).to(dtype)
    snd = torch.randint(0, N, (Z,), generator=g).to(index_dtype)
    rcv = torch.randint(0, N, (Z,), generator=g).to(index_dtype)
    if sort_receivers:
        rcv = torch.sort(rcv)[0]
    cot = torch.randn(N, D3, dtype=torch.float64, generator=g).to(dtype)
    a = [t.clone().requires_grad_(True) for t in (w, x1, x2)]
    ref = naive_segmented_polynomial(spec, a, {1: snd}, {0: N}, {0: rcv})[0]
    ref_grads = torch.autograd.grad((ref * cot).sum(), a)
    b = [t.clone().to(device).requires_grad_(True) for t in (w, x1, x2)]
    out = m(b[1], b[2], b[0], indices_1=snd.to(device), indices_out=rcv.to(device), size_out=N)
    grads = torch.autograd.grad(out, b, cot.to(device))
    tol = tol or TOL[dtype]
    assert_close(out, ref, tol, "out")
    for name, p, q in zip(("dw", "dx1", "dx2"), ref_grads, grads):
        assert_close(q, p, tol, name)
    return out, grads


# --------------------------------------------------------------------------- channel-wise configurations
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_cfg1_channelwise_batch4096(device, dtype):
    """Config 1: 32x0e+32x1o+32x2e (x) 0e+1o+2e, batch 4096, all operands batched, forward + three gradients."""
    m = cw_module("32x0e+32x1o+32x2e", "0e+1o+2e", "0e+1o+2e")
    spec = spec_from_polynomial(m.f._polynomial_orig)
    g = torch.Generator().manual_seed(0)
    Z = 4096
    x1, x2, w = (torch.randn(Z, n, dtype=torch.float64, generator=g).to(dtype) for n in (288, 9, 352))
    cot = torch.randn(Z, 1120, dtype=torch.float64, generator=g).to(dtype)
    a = [t.clone().requires_grad_(True) for t in (w, x1, x2)]
    ref = naive_segmented_polynomial(spec, a)[0]
    ref_grads = torch.autograd.grad((ref * cot).sum(), a)
    b = [t.clone().to(device).requires_grad_(True) for t in (w, x1, x2)]
    out = m(b[1], b[2], b[0])
    grads = torch.autograd.grad(out, b, cot.to(device))
    plan = m.f.m._plan(dtype)
    assert plan.specialised(device) and plan.backward_plan((True, True, True)).specialised(device)
    assert_close(out, ref, TOL[dtype], "out")
    for name, p, q in zip(("dw", "dx1", "dx2"), ref_grads, grads):
        assert_close(q, p, TOL[dtype], name)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("deterministic", ["0", "1"])
def test_cfg2_reduced_indexed_channelwise(device, dtype, deterministic, monkeypatch):
    """Config 2 descriptor (128 channels, l <= 3) on 300 nodes / 4000 edges; both scatter policies of dx1."""
    monkeypatch.setenv("CUEQ_DETERMINISTIC", deterministic)
    m = cw_module("128x0e+128x1o+128x2e+128x3o", "0e+1o+2e+3o", "0e+1o+2e+3o")
    run_cw_case(device, m, N=300, Z=4000, dtype=dtype, seed=1)
    assert m.f.m._plan(dtype).specialised(device)


@pytest.mark.parametrize("forced_generic", ["", "1"])
def test_channelwise_unsorted_receivers_int64_and_empty_rows(device, forced_generic, monkeypatch):
    if forced_generic:
        monkeypatch.setenv("CUEQ_FORCE_GENERIC", "1")
    m = cw_module("32x0e+32x1o+32x2e", "0e+1o+2e", "0e+1o+2e")
    # N much larger than Z: most output rows receive nothing and must come out as zeros
    out, _ = run_cw_case(device, m, N=500, Z=64, dtype=torch.float64, seed=2, sort_receivers=False,
                         index_dtype=torch.int64)
    assert (out.abs().sum(1) == 0).sum().item() >= 500 - 64


def test_channelwise_non_registered_descriptor_uses_table_driven_kernels(device):
    # 48 channels (not a multiple of the wavefront size), mixed parities, a filter that drops irreps
    m = cw_module("48x0e+48x1o+48x1e", "0e+1o+2e", "0e+1o+1e+2o")
    run_cw_case(device, m, N=40, Z=333, dtype=torch.float64, seed=3)
    run_cw_case(device, m, N=40, Z=333, dtype=torch.float32, seed=3)
    from cuequivariance_amd import jit

    if not jit.enabled():  # (with compilation at first use left on, the descriptor gets kernels of its own)
        assert not m.f.m._plan(torch.float32).specialised(device)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_table_driven_kernels_split_very_long_output_rows(device, dtype, monkeypatch):
    """Three output rows that collect 1 400 edges each (a gradient indexed by a handful of classes looks like this): the
    table-driven kernels work on such a row in pieces of its edge range and add the pieces in order.  48 and 96 channels
    (one wavefront per 64 channels of a row segment, the second one partly filled), every gradient, twice for the same bits."""
    monkeypatch.setenv("CUEQ_FORCE_GENERIC", "1")
    for channels in (48, 96):
        m = cw_module(f"{channels}x0e+{channels}x1o", "0e+1o", "0e+1o")
        out, grads = run_cw_case(device, m, N=3, Z=4200, dtype=dtype, seed=11 + channels, sort_receivers=False)
        out2, grads2 = run_cw_case(device, m, N=3, Z=4200, dtype=dtype, seed=11 + channels, sort_receivers=False)
        assert torch.equal(out, out2) and all(torch.equal(a, b) for a, b in zip(grads, grads2))


def test_channelwise_mul_ir_layout_and_shared_internal_weights(device):
    from cuequivariance_amd import cuet

    irreps1, irreps2 = cue.Irreps("O3", "8x0e+8x1o"), cue.Irreps("O3", "0e+1o")
    torch.manual_seed(0)
    m_ir = cuet.ChannelWiseTensorProduct(irreps1, irreps2, "0e+1o", layout=cue.ir_mul, device=device, dtype=torch.float64)
    m_mul = cuet.ChannelWiseTensorProduct(irreps1, irreps2, "0e+1o", layout=cue.mul_ir, device=device, dtype=torch.float64)
    with torch.no_grad():
        m_mul.weight.copy_(m_ir.weight)
    Z = 50
    x1 = torch.randn(Z, irreps1.dim, dtype=torch.float64, device=device)
    x2 = torch.randn(Z, irreps2.dim, dtype=torch.float64, device=device)

    def to_mul_ir(x, irreps):
        outs, off = [], 0
        for mul, ir in irreps:
            outs.append(x[:, off: off + mul * ir.dim].reshape(Z, ir.dim, mul).transpose(1, 2).reshape(Z, -1))
            off += mul * ir.dim
        return torch.cat(outs, 1)

    y_ir = m_ir(x1, x2)
    y_mul = m_mul(to_mul_ir(x1, irreps1), to_mul_ir(x2, irreps2))
    assert_close(y_mul, to_mul_ir(y_ir, m_ir.irreps_out), 1e-13, "layouts")
    # shared weights: the oracle with a one-row weight
    spec = spec_from_polynomial(m_ir.f._polynomial_orig)
    ref = naive_segmented_polynomial(spec, [m_ir.weight.detach().cpu(), x1.cpu(), x2.cpu()])[0]
    assert_close(y_ir, ref, 1e-12, "shared weights")
    (y_ir.square().sum()).backward()
    w = m_ir.weight.detach().cpu().clone().requires_grad_(True)
    naive_segmented_polynomial(spec, [w, x1.cpu(), x2.cpu()])[0].square().sum().backward()
    assert_close(m_ir.weight.grad, w.grad, 1e-12, "dw shared")


# --------------------------------------------------------------------------- full-size properties
def test_cfg2_full_size_properties(device, monkeypatch):
    """100k edges / 5k nodes: linearity, agreement of the two independent kernel families, reproducibility."""
    m = cw_module("128x0e+128x1o+128x2e+128x3o", "0e+1o+2e+3o", "0e+1o+2e+3o")
    g = torch.Generator().manual_seed(7)
    N, E = 5000, 100_000
    x1 = torch.randn(N, 2048, generator=g).to(device)
    x2 = torch.randn(E, 16, generator=g).to(device)
    w1, w2 = torch.randn(E, 2944, generator=g).to(device), torch.randn(E, 2944, generator=g).to(device)
    snd = torch.randint(0, N, (E,), generator=g, dtype=torch.int32).to(device)
    rcv = torch.sort(torch.randint(0, N, (E,), generator=g, dtype=torch.int32))[0].to(device)
    cot = torch.randn(N, 12672, generator=g).to(device)

    def f(w, x1_=x1):
        return m(x1_, x2, w, indices_1=snd, indices_out=rcv, size_out=N)

    y1, y2, y12 = f(w1), f(w2), f(w1 + w2)
    assert_close(y12, y1 + y2, 1e-5, "linearity in w")
    assert_close(f(w1, 2.0 * x1), 2.0 * y1, 1e-5, "homogeneity in x1")
    assert torch.equal(f(w1), y1), "forward must be bit-reproducible"

    def grads(w):
        ws, xs, x2s = w.clone().requires_grad_(True), x1.clone().requires_grad_(True), x2.clone().requires_grad_(True)
        out = m(xs, x2s, ws, indices_1=snd, indices_out=rcv, size_out=N)
        return out, torch.autograd.grad(out, [ws, xs, x2s], cot)

    out_s, g_s = grads(w1)
    monkeypatch.setenv("CUEQ_DETERMINISTIC", "1")
    _, g_d1 = grads(w1)
    _, g_d2 = grads(w1)
    for a, b in zip(g_d1, g_d2):
        assert torch.equal(a, b), "deterministic backward must be bit-reproducible"
    for name, a, b in zip(("dw", "dx1", "dx2"), g_s, g_d1):
        assert_close(a, b, 1e-5, f"atomic vs ordered scatter {name}")
    # the table-driven kernels are an independent implementation of the same tables
    monkeypatch.setenv("CUEQ_FORCE_GENERIC", "1")
    out_g, g_g = grads(w1)
    assert_close(out_s, out_g, 1e-5, "specialised vs table-driven out")
    for name, a, b in zip(("dw", "dx1", "dx2"), g_s, g_g):
        assert_close(a, b, 1e-5, f"specialised vs table-driven {name}")
    # <cot, f(w)> is linear in w: its gradient w.r.t. w dotted with w gives it back (Euler)
    lhs = (out_s.double() * cot.double()).sum().item()
    rhs = (g_s[0].double() * w1.double()).sum().item()
    assert abs(lhs - rhs) <= 1e-5 * max(abs(lhs), (out_s.double().abs() * cot.double().abs()).sum().item())


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("deterministic", ["0", "1"])
def test_cfg2_full_size_block_of_receivers_against_oracle(device, dtype, deterministic, monkeypatch):
    """The benchmark's own problem (5 000 nodes, 100 000 edges, 128 channels, l <= 3) against the oracle on 200 contiguous
    receiver rows: the output rows of the block depend only on the block's edges (all senders), and with a cotangent
    that is zero outside the block so do all three gradients - dw and dx2 on the block's edges (exactly zero elsewhere)
    and dx1 on every node.  The oracle evaluates just those edges; the GPU runs the whole problem in one call."""
    monkeypatch.setenv("CUEQ_DETERMINISTIC", deterministic)
    m = cw_module("128x0e+128x1o+128x2e+128x3o", "0e+1o+2e+3o", "0e+1o+2e+3o")
    spec = spec_from_polynomial(m.f._polynomial_orig)
    g = torch.Generator().manual_seed(11)
    N, E, r0, r1 = 5000, 100_000, 2417, 2617
    x1 = torch.randn(N, 2048, generator=g).to(dtype)
    x2 = torch.randn(E, 16, generator=g).to(dtype)
    w = torch.randn(E, 2944, generator=g).to(dtype)
    snd = torch.randint(0, N, (E,), generator=g, dtype=torch.int32)
    rcv = torch.sort(torch.randint(0, N, (E,), generator=g, dtype=torch.int32))[0]
    cot = torch.zeros(N, 12672, dtype=dtype)
    cot[r0:r1] = torch.randn(r1 - r0, 12672, generator=g).to(dtype)
    sel = ((rcv >= r0) & (rcv < r1)).nonzero().squeeze(1)
    assert 3000 < sel.numel() < 5000 and torch.equal(sel, torch.arange(sel[0], sel[-1] + 1))
    # oracle: the block's edges only, receivers renumbered to [0, 200)
    a = [w[sel].clone().requires_grad_(True), x1.clone().requires_grad_(True), x2[sel].clone().requires_grad_(True)]
    ref = naive_segmented_polynomial(spec, a, {1: snd[sel]}, {0: r1 - r0}, {0: rcv[sel] - r0})[0]
    ref_dw, ref_dx1, ref_dx2 = torch.autograd.grad(ref, a, cot[r0:r1])
    # GPU: the whole problem
    b = [t.clone().to(device).requires_grad_(True) for t in (w, x1, x2)]
    out = m(b[1], b[2], b[0], indices_1=snd.to(device), indices_out=rcv.to(device), size_out=N)
    dw, dx1, dx2 = torch.autograd.grad(out, b, cot.to(device))
    assert m.f.m._plan(dtype).specialised(device)
    tol = TOL[dtype]
    assert_close(out[r0:r1], ref, tol, "out rows of the block")
    assert_close(dw[sel.to(device)], ref_dw, tol, "dw of the block's edges")
    assert_close(dx2[sel.to(device)], ref_dx2, tol, "dx2 of the block's edges")
    assert_close(dx1, ref_dx1, tol, "dx1 (all nodes)")
    outside = torch.ones(E, dtype=torch.bool)
    outside[sel] = False
    assert dw[outside.to(device)].abs().max().item() == 0 and dx2[outside.to(device)].abs().max().item() == 0


# --------------------------------------------------------------------------- indexing matrix (table-driven kernels)
def small_poly():
    e = cue.descriptors.channelwise_tensor_product(
        cue.Irreps("O3", "16x0e + 16x1o"), cue.Irreps("O3", "0e + 1o + 2e"), cue.Irreps("O3", "0e + 1o")
    )
    return e.polynomial


MODES = ["shared", "batched", "indexed"]


@pytest.mark.parametrize("modes", [c for c in itertools.product(MODES, repeat=3)
                                   if c in {("batched",) * 3, ("shared", "batched", "batched"),
                                            ("shared", "indexed", "batched"), ("indexed", "indexed", "indexed"),
                                            ("batched", "shared", "batched"), ("batched", "indexed", "shared"),
                                            ("indexed", "batched", "batched"), ("shared", "shared", "batched"),
                                            ("batched", "batched", "indexed")}])
@pytest.mark.parametrize("out_mode", ["batched", "indexed", "shared"])
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_indexing_matrix_forward_and_gradients(device, modes, out_mode, dtype):
    from cuequivariance_amd import cuet

    poly = small_poly()
    spec = spec_from_polynomial(poly)
    mod = cuet.SegmentedPolynomial(poly, method="uniform_1d")
    g = torch.Generator().manual_seed(hash((modes, out_mode)) % 1000)
    Z, R = 37, 11
    inputs, idx_in = [], {}
    for k, (mode, op) in enumerate(zip(modes, poly.inputs)):
        rows = {"shared": 1, "batched": Z, "indexed": R}[mode]
        inputs.append(torch.randn(rows, op.size, dtype=torch.float64, generator=g).to(dtype))
        if mode == "indexed":
            idx_in[k] = torch.sort(torch.randint(0, R, (Z,), generator=g, dtype=torch.int32))[0]
    out_shapes, out_idx = {}, {}
    if out_mode == "indexed":
        out_idx[0] = torch.randint(0, R, (Z,), generator=g, dtype=torch.int32)
        out_shapes[0] = R
    elif out_mode == "shared":
        out_shapes[0] = 1
    out_rows = out_shapes.get(0, Z)
    cot = torch.randn(out_rows, poly.outputs[0].size, dtype=torch.float64, generator=g).to(dtype)

    a = [t.clone().requires_grad_(True) for t in inputs]
    ref = naive_segmented_polynomial(spec, a, idx_in, out_shapes, out_idx)[0]
    ref_grads = torch.autograd.grad((ref * cot).sum(), a)
    b = [t.clone().to(device).requires_grad_(True) for t in inputs]
    out = mod(
        b,
        {k: v.to(device) for k, v in idx_in.items()},
        {k: torch.empty(v, 1, device="meta") for k, v in out_shapes.items()},
        {k: v.to(device) for k, v in out_idx.items()},
    )[0]
    grads = torch.autograd.grad(out, b, cot.to(device))
    assert_close(out, ref, TOL[dtype], "out")
    for k, (p, q) in enumerate(zip(ref_grads, grads)):
        assert_close(q, p, TOL[dtype], f"grad {k}")


@pytest.mark.parametrize("io,math", [(torch.bfloat16, torch.float32), (torch.float16, torch.float32),
                                     (torch.float32, torch.float64), (torch.bfloat16, None)])
def test_low_precision_io(device, io, math):
    from cuequivariance_amd import cuet

    poly = small_poly()
    spec = spec_from_polynomial(poly)
    mod = cuet.SegmentedPolynomial(poly, method="uniform_1d", math_dtype=math)
    g = torch.Generator().manual_seed(5)
    Z = 64
    inputs = [torch.randn(Z, op.size, generator=g).to(io) for op in poly.inputs]
    # the oracle in float64 on the rounded inputs is the reference value; the kernel accumulates in the math dtype
    ref = naive_segmented_polynomial(spec, [t.double() for t in inputs])[0]
    out = mod([t.to(device) for t in inputs])[0]
    assert out.dtype == io
    assert_close(out, ref, TOL[io], "out")


def test_second_derivative(device):
    from cuequivariance_amd import cuet

    poly = small_poly()
    spec = spec_from_polynomial(poly)
    mod = cuet.SegmentedPolynomial(poly, method="uniform_1d")
    g = torch.Generator().manual_seed(9)
    Z, R = 23, 7
    inputs = [torch.randn(rows, op.size, dtype=torch.float64, generator=g)
              for rows, op in zip((Z, R, Z), poly.inputs)]
    snd = torch.randint(0, R, (Z,), generator=g, dtype=torch.int32)
    rcv = torch.randint(0, R, (Z,), generator=g, dtype=torch.int32)

    def scalar(fn, ins, dev):
        out = fn(ins, dev)
        gs = torch.autograd.grad(out.square().sum(), ins, create_graph=True)
        return sum((gi.sin()).sum() for gi in gs)

    a = [t.clone().requires_grad_(True) for t in inputs]
    b = [t.clone().to(device).requires_grad_(True) for t in inputs]
    ra = scalar(lambda ins, _: naive_segmented_polynomial(spec, ins, {1: snd}, {0: R}, {0: rcv})[0], a, None)
    rb = scalar(lambda ins, d: mod(ins, {1: snd.to(d)}, {0: torch.empty(R, 1, device="meta")}, {0: rcv.to(d)})[0], b, device)
    ga, gb = torch.autograd.grad(ra, a), torch.autograd.grad(rb, b)
    assert_close(rb.reshape(1), ra.reshape(1), 1e-12, "scalar")
    for k, (p, q) in enumerate(zip(ga, gb)):
        assert_close(q, p, 1e-11, f"second-order grad {k}")


def test_repeated_buffer_polynomial(device):
    """Degree-2 and degree-3 operations reading the same buffer several times (symmetric-contraction shape)."""
    from cuequivariance_amd import cuet

    u = 8
    g = torch.Generator().manual_seed(11)
    ops = []
    wseg = 0
    x_op = cue.SegmentedOperand([(u,)] * 4)
    stps = []
    for degree in (1, 2, 3):
        d = cue.SegmentedTensorProduct.from_subscripts(",".join(["u"] * (degree + 2)))
        stps.append(d)
    # weights: 6 segments shared by the three operations
    for d, degree in zip(stps, (1, 2, 3)):
        d.add_segments(0, [(u,)] * 6)
        for k in range(1, degree + 1):
            d.add_segments(k, [(u,)] * 4)
        d.add_segments(degree + 1, [(u,)] * 2)
        for _ in range(5):
            idx = [int(torch.randint(0, 6, (1,), generator=g))] + \
                  [int(torch.randint(0, 4, (1,), generator=g)) for _ in range(degree)] + \
                  [int(torch.randint(0, 2, (1,), generator=g))]
            d.add_path(*idx, c=float(torch.randn(1, generator=g)))
        ops.append((cue.Operation([0] + [1] * degree + [2]), d))
    poly = cue.SegmentedPolynomial([stps[0].operands[0], x_op], [stps[0].operands[-1]], ops)
    spec = spec_from_polynomial(poly)
    mod = cuet.SegmentedPolynomial(poly, method="uniform_1d")
    Z, C = 29, 3
    w = torch.randn(C, 6 * u, dtype=torch.float64, generator=g)
    x = torch.randn(Z, 4 * u, dtype=torch.float64, generator=g)
    species = torch.randint(0, C, (Z,), generator=g, dtype=torch.int32)
    cot = torch.randn(Z, 2 * u, dtype=torch.float64, generator=g)
    a = [w.clone().requires_grad_(True), x.clone().requires_grad_(True)]
    ref = naive_segmented_polynomial(spec, a, {0: species})[0]
    rg = torch.autograd.grad((ref * cot).sum(), a)
    b = [w.clone().to(device).requires_grad_(True), x.clone().to(device).requires_grad_(True)]
    out = mod(b, {0: species.to(device)})[0]
    gg = torch.autograd.grad(out, b, cot.to(device))
    assert_close(out, ref, 1e-12, "out")
    assert_close(gg[0], rg[0], 1e-12, "dw (scatter over species)")
    assert_close(gg[1], rg[1], 1e-12, "dx")


def test_empty_batch_and_functional_entry_point(device):
    from cuequivariance_amd import cuet
    from cuequivariance_amd.cuet.uniform_1d import BATCH_DIM_AUTO, BATCH_DIM_INDEXED, uniform_1d

    poly = small_poly()
    t = U1dTables.from_polynomial(poly.flatten_coefficient_modes().squeeze_modes())
    spec = spec_from_polynomial(poly)
    g = torch.Generator().manual_seed(13)
    Z, R = 19, 5
    w = torch.randn(Z, t.width(0), dtype=torch.float64, generator=g)
    x1 = torch.randn(R, t.width(1), dtype=torch.float64, generator=g)
    x2 = torch.randn(Z, t.width(2), dtype=torch.float64, generator=g)
    snd = torch.randint(0, R, (Z,), generator=g, dtype=torch.int64)
    rcv = torch.randint(0, R, (Z,), generator=g, dtype=torch.int64)
    ref = naive_segmented_polynomial(spec, [w, x1, x2], {1: snd}, {0: R}, {0: rcv})[0]
    # the 21-argument operator, called the way the reference's frontend calls its closed op
    out = uniform_1d(
        "test", torch.float64, t.operand_extent, t.num_inputs, t.num_outputs, 2, list(t.buffer_dim),
        list(t.buffer_num_segments), [BATCH_DIM_AUTO, BATCH_DIM_INDEXED, BATCH_DIM_AUTO, BATCH_DIM_INDEXED],
        [-1, 0, -1, 1, R, R], list(t.dtypes), len(t.num_operands), list(t.num_operands), list(t.operations),
        list(t.num_paths), list(t.path_indices_start), list(t.path_coefficients_start), list(t.path_indices),
        list(t.path_coefficients), BATCH_DIM_AUTO,
        [w.to(device), x1.to(device), x2.to(device), snd.to(device), rcv.to(device)],
    )[0]
    assert_close(out, ref, 1e-12, "functional op")
    # empty batch: indexed output is all zeros, batched output has zero rows
    mod = cuet.SegmentedPolynomial(poly, method="uniform_1d")
    e = torch.empty(0, dtype=torch.int32, device=device)
    out = mod([w[:0].to(device), x1.to(device), x2[:0].to(device)], {1: e}, {0: torch.empty(R, 1, device="meta")}, {0: e})[0]
    assert out.shape == (R, t.width(3)) and out.abs().sum().item() == 0
    out = mod([w[:0].to(device), x1[:0].to(device), x2[:0].to(device)])[0]
    assert out.shape == (0, t.width(3))
    with pytest.raises(RuntimeError):
        mod([w, x1[snd], x2])  # CPU tensors are rejected, there is no CPU path
    with pytest.raises(ValueError):
        cuet.SegmentedPolynomial(poly, method="naive")


@pytest.mark.parametrize("sorted_ids", [True, False])
@pytest.mark.parametrize("index_dtype", [torch.int32, torch.int64])
def test_segment_csr_bit_exact(device, sorted_ids, index_dtype):
    from cuequivariance_amd.cuet.uniform_1d import _segment_csr

    g = torch.Generator().manual_seed(17)
    n, nrows = 10_000, 777
    ids = torch.randint(0, nrows, (n,), generator=g).to(index_dtype)
    if sorted_ids:
        ids = torch.sort(ids)[0]
    offsets, perm = _segment_csr(ids.to(device), nrows)
    exp_perm = torch.sort(ids.long(), stable=True)[1]
    exp_offsets = torch.zeros(nrows + 1, dtype=torch.int64)
    exp_offsets[1:] = torch.cumsum(torch.bincount(ids.long(), minlength=nrows), 0)
    assert torch.equal(offsets.cpu(), exp_offsets)
    assert torch.equal(perm.cpu()[:n], exp_perm)
    with pytest.raises(Exception):
        _segment_csr(torch.tensor([0, nrows], dtype=index_dtype, device=device), nrows)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_spherical_harmonics_module(device, dtype):
    """``cuet.SphericalHarmonics`` (reference ``operations/spherical_harmonics.py:26-93``): values and the gradient
    with respect to the vectors against the oracle, with and without normalisation."""
    from cuequivariance_amd import cuet

    ls = [0, 1, 2, 3]
    g = torch.Generator().manual_seed(0)
    v = torch.randn(301, 3, dtype=torch.float64, generator=g).to(dtype)
    cot = torch.randn(301, 16, dtype=torch.float64, generator=g).to(dtype)
    for normalize in (True, False):
        m = cuet.SphericalHarmonics(ls, normalize=normalize)
        spec = spec_from_polynomial(m.f._polynomial_orig)
        a = v.clone().requires_grad_(True)
        vin = torch.nn.functional.normalize(a, dim=1) if normalize else a
        ref = naive_segmented_polynomial(spec, [vin])[0]
        (ref_grad,) = torch.autograd.grad(ref, [a], cot)
        b = v.clone().to(device).requires_grad_(True)
        out = m(b)
        (grad,) = torch.autograd.grad(out, [b], cot.to(device))
        assert_close(out, ref, TOL[dtype], "Y")
        assert_close(grad, ref_grad, 4 * TOL[dtype], "dY/dx")


@pytest.mark.gpu
def test_gradient_subset_runs_on_the_specialised_full_backward(device):
    """Only x1 and x2 ask for gradients (weights fixed, as in inference with forces): there are no specialised kernels for
    that subset, so the specialised kernels for all three gradients run and the unwanted one is dropped; against the
    oracle."""
    from cuequivariance_amd.cuet.uniform_1d import _backward_choice

    m = cw_module("32x0e+32x1o+32x2e", "0e+1o+2e", ["0e", "1o", "2e"])
    spec = spec_from_polynomial(m.f._polynomial_orig)
    g = torch.Generator().manual_seed(77)
    N, Z = 40, 600
    x1 = torch.randn(N, m.irreps_in1.dim, generator=g)
    x2 = torch.randn(Z, m.irreps_in2.dim, generator=g)
    w = torch.randn(Z, m.weight_numel, generator=g)
    snd = torch.randint(0, N, (Z,), generator=g, dtype=torch.int32)
    rcv = torch.sort(torch.randint(0, N, (Z,), generator=g, dtype=torch.int32))[0]
    cot = torch.randn(N, m.irreps_out.dim, generator=g)
    a = [w.clone(), x1.clone().requires_grad_(True), x2.clone().requires_grad_(True)]
    ref = naive_segmented_polynomial(spec, a, {1: snd}, {0: N}, {0: rcv})[0]
    ref_grads = torch.autograd.grad(ref, a[1:], cot)
    b = [w.to(device), x1.to(device).requires_grad_(True), x2.to(device).requires_grad_(True)]
    out = m(b[1], b[2], b[0], indices_1=snd.to(device), indices_out=rcv.to(device), size_out=N)
    grads = torch.autograd.grad(out, b[1:], cot.to(device))
    for name, p, q in zip(("dx1", "dx2"), ref_grads, grads):
        assert_close(q, p, 1e-5, name)
    plan = m.f.m._plan(torch.float32)
    from cuequivariance_amd import jit

    chosen, computed = _backward_choice(plan, (False, True, True), device)
    assert chosen.specialised(device) and computed == (True, True, True)
    if not jit.enabled():  # (with kernels compiled at first use the subset would get a unit of its own)
        assert not plan.backward_plan((False, True, True)).specialised(device)
