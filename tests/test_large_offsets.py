"""Element offsets beyond 2^31: one call over a batch whose largest operand holds more than 2^31 elements against the
same work done in two halves (each below 2^31).  Size-independent properties only - the oracle would take hours here:
batched outputs and per-row gradients of the halves concatenate, indexed outputs and shared gradients add."""

import gc

import pytest
import torch

from cuequivariance_amd import cue

pytestmark = pytest.mark.gpu


def _close(got, want, name):
    scale = want.abs().max().item()
    err = (got - want).abs().max().item()
    assert err <= 1e-5 * scale, (name, err, scale)


@pytest.fixture(autouse=True)
def _release():
    yield
    gc.collect()
    torch.cuda.empty_cache()


def test_channelwise_indexed_weights_beyond_2g_elements(device):
    """128 channels, l <= 3, 2 000 nodes, 800 000 edges: the per-edge weights hold 2.36e9 elements."""
    from cuequivariance_amd import cuet

    i1 = cue.Irreps("O3", "128x0e+128x1o+128x2e+128x3o")
    i2 = cue.Irreps("O3", "0e+1o+2e+3o")
    m = cuet.ChannelWiseTensorProduct(i1, i2, "0e+1o+2e+3o", layout=cue.ir_mul, shared_weights=False)
    N, E = 2000, 800_000
    assert E * m.weight_numel > 2 ** 31
    g = torch.Generator(device=device).manual_seed(0)
    x1 = torch.randn(N, i1.dim, device=device, generator=g)
    x2 = torch.randn(E, i2.dim, device=device, generator=g)
    w = torch.randn(E, m.weight_numel, device=device, generator=g)
    snd = torch.randint(0, N, (E,), device=device, generator=g, dtype=torch.int32)
    rcv = torch.sort(torch.randint(0, N, (E,), device=device, generator=g, dtype=torch.int32))[0]
    cot = torch.randn(N, m.irreps_out.dim, device=device, generator=g)

    def run(lo, hi):
        a = [x1.clone().requires_grad_(True), x2[lo:hi].requires_grad_(True), w[lo:hi].requires_grad_(True)]
        out = m(a[0], a[1], a[2], indices_1=snd[lo:hi], indices_out=rcv[lo:hi], size_out=N)
        return (out.detach(),) + torch.autograd.grad(out, a, cot)

    out, dx1, dx2, dw = run(0, E)
    h = E // 2
    out_a, dx1_a, dx2_a, dw_a = run(0, h)
    _close(dw[:h], dw_a, "dw, first half")
    _close(dx2[:h], dx2_a, "dx2, first half")
    del dw_a, dx2_a
    out_b, dx1_b, dx2_b, dw_b = run(h, E)
    _close(dw[h:], dw_b, "dw, second half")  # rows whose element offset exceeds 2^31
    _close(dx2[h:], dx2_b, "dx2, second half")
    _close(out, out_a + out_b, "out")
    _close(dx1, dx1_a + dx1_b, "dx1")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear_rows_beyond_2g_elements(device, dtype):
    """Linear on 128x0e+128x1o+128x2e (1152 columns), 2 000 000 rows: 2.3e9 elements per operand."""
    from cuequivariance_amd import cuet

    irreps = cue.Irreps("O3", "128x0e+128x1o+128x2e")
    m = cuet.Linear(irreps, irreps, layout=cue.ir_mul, internal_weights=False, method="fused_tp")
    Z = 2_000_000
    assert Z * irreps.dim > 2 ** 31
    g = torch.Generator(device=device).manual_seed(1)
    x = torch.randn(Z, irreps.dim, device=device, generator=g).to(dtype)
    w = torch.randn(1, m.weight_numel, device=device, generator=g).to(dtype)
    cot = torch.randn(Z, irreps.dim, device=device, generator=g).to(dtype)

    def run(lo, hi):
        a = [x[lo:hi].requires_grad_(True), w.clone().requires_grad_(True)]
        out = m(a[0], a[1])
        return (out.detach(),) + torch.autograd.grad(out, a, cot[lo:hi])

    out, dx, dw = run(0, Z)
    h = Z // 2
    out_a, dx_a, dw_a = run(0, h)
    out_b, dx_b, dw_b = run(h, Z)
    # per-row results do not depend on the batch they are computed in
    assert torch.equal(out[:h], out_a) and torch.equal(out[h:], out_b)
    assert torch.equal(dx[:h], dx_a) and torch.equal(dx[h:], dx_b)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    want = dw_a.double() + dw_b.double()
    assert (dw.double() - want).abs().max().item() <= tol * want.abs().max().item()


def test_symmetric_contraction_rows_beyond_2g_elements(device):
    """Degree-3 contraction of 128x(0e+1o+2e+3o) (2048 columns) on 1 100 000 nodes: 2.25e9 input elements."""
    from cuequivariance_amd import cuet

    irreps_in = cue.Irreps("O3", "128x0e+128x1o+128x2e+128x3o")
    irreps_out = cue.Irreps("O3", "128x0e+128x1o")
    m = cuet.SymmetricContraction(irreps_in, irreps_out, 3, 10, layout_in=cue.ir_mul, layout_out=cue.ir_mul,
                                  dtype=torch.float32, device=device)
    Z = 1_100_000
    assert Z * irreps_in.dim > 2 ** 31
    g = torch.Generator(device=device).manual_seed(2)
    x = torch.randn(Z, irreps_in.dim, device=device, generator=g) * 0.5
    idx = torch.randint(0, 10, (Z,), device=device, generator=g, dtype=torch.int32)
    cot = torch.randn(Z, irreps_out.dim, device=device, generator=g)

    def run(lo, hi):
        a = x[lo:hi].requires_grad_(True)
        out = m(a, idx[lo:hi])
        dx, dw = torch.autograd.grad(out, [a, m.weight], cot[lo:hi])
        return out.detach(), dx, dw

    out, dx, dw = run(0, Z)
    h = Z // 2
    out_a, dx_a, dw_a = run(0, h)
    out_b, dx_b, dw_b = run(h, Z)
    _close(out[:h], out_a, "out, first half")
    _close(out[h:], out_b, "out, second half")
    _close(dx[:h], dx_a, "dx, first half")
    _close(dx[h:], dx_b, "dx, second half")
    _close(dw, dw_a + dw_b, "dw")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_transpose_more_row_tiles_than_grid_y_holds(device, dtype):
    """4 194 368 rows of 8 and of 6 columns (one more 64-row tile than grid.y can index, even and odd column pairs):
    bit-exact against a strided copy, both ways."""
    from cuequivariance_amd.cuet import triangle as T

    for cols in (8, 6, 5):
        rows = 65536 * 64 + 64
        x = torch.randn(rows, cols, device=device).to(dtype)
        y = T.transpose(x)
        assert torch.equal(y, x.t().contiguous())
        assert torch.equal(T.transpose(y), x)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_triangle_update_more_pair_rows_than_one_launch_takes(device, dtype):
    """Two pair tensors of 2048 x 2048 x 128 in one call: 8 388 608 pair rows, more than the projections' launches take
    at once (their row tiles sit on grid.y), so they run in slabs of rows.  Batch elements are independent: each half of the output and of
    the input gradient must be what a call on that batch element alone gives; weight gradients add."""
    from cuequivariance_amd.cuet import triangle_multiplicative_update as tmu

    B, N, D = 2, 2048, 128
    g = torch.Generator(device=device).manual_seed(5)
    ws = {k: (torch.randn(*shape, device=device, generator=g) * 0.09).to(dtype)
          for k, shape in (("p_in_weight", (2 * D, D)), ("g_in_weight", (2 * D, D)), ("p_out_weight", (D, D)), ("g_out_weight", (D, D)))}
    x = torch.randn(B, N, N, D, device=device, generator=g).to(dtype)
    mask = (torch.rand(B, N, N, device=device, generator=g) > 0.1).to(dtype)
    cot = torch.randn(B, N, N, D, device=device, generator=g).to(dtype)

    def run(lo, hi):
        a = x[lo:hi].requires_grad_(True)
        w = {k: v.clone().requires_grad_(True) for k, v in ws.items()}
        out = tmu(a, "outgoing", mask=mask[lo:hi], **w)
        grads = torch.autograd.grad(out, [a] + list(w.values()), cot[lo:hi])
        return out.detach(), grads[0], [t.float() for t in grads[1:]]

    tol = 1e-5 if dtype == torch.float32 else 2e-2
    out, dx, dws = run(0, B)
    sums = [torch.zeros_like(t) for t in dws]
    for b in range(B):
        o, d, dw = run(b, b + 1)
        for name, u, v in (("out", out[b:b + 1], o), ("dx", dx[b:b + 1], d)):
            err = (u.float() - v.float()).abs().max().item()
            assert err <= tol * v.float().abs().max().item(), (name, b, err)
        for s_, t in zip(sums, dw):
            s_ += t
        del o, d, dw
    for name, u, v in zip(ws, dws, sums):
        assert (u - v).abs().max().item() <= tol * v.abs().max().item(), name


@pytest.mark.parametrize("kind", ["linear", "fully_connected"])
def test_dense_more_rows_than_one_launch_takes(device, kind):
    """9 000 000 rows through the table-driven GEMM launches of the dense executor (row tiles on grid.y: 8 355 840 rows a
    launch, the rest in a second slab): per-row results equal those of the two halves, weight gradients add."""
    from cuequivariance_amd import cuet

    Z = 9_000_000
    g = torch.Generator(device=device).manual_seed(6)
    if kind == "linear":
        irreps = cue.Irreps("O3", "32x0e+32x1o")
        m = cuet.Linear(irreps, irreps, layout=cue.ir_mul, internal_weights=False, method="fused_tp")
        ins = [torch.randn(Z, irreps.dim, device=device, generator=g)]
        call = lambda a, w: m(a[0], w)
    else:
        i1, i2 = cue.Irreps("O3", "8x0e+8x1o"), cue.Irreps("O3", "0e+1o")
        m = cuet.FullyConnectedTensorProduct(i1, i2, i1, layout=cue.ir_mul, internal_weights=False)
        ins = [torch.randn(Z, i1.dim, device=device, generator=g), torch.randn(Z, i2.dim, device=device, generator=g)]
        call = lambda a, w: m(a[0], a[1], w)
    w0 = torch.randn(1, m.weight_numel, device=device, generator=g)
    cot = torch.randn(Z, m.irreps_out.dim, device=device, generator=g)

    def run(lo, hi):
        a = [t[lo:hi].requires_grad_(True) for t in ins]
        w = w0.clone().requires_grad_(True)
        out = call(a, w)
        grads = torch.autograd.grad(out, a + [w], cot[lo:hi])
        return [out.detach()] + list(grads[:-1]), grads[-1]

    rows, dw = run(0, Z)
    h = Z // 2
    total = torch.zeros_like(dw, dtype=torch.float64)
    for lo, hi in ((0, h), (h, Z)):
        r, d = run(lo, hi)
        for u, v in zip(rows, r):
            assert torch.equal(u[lo:hi], v)
        total += d.double()
        del r, d
    assert (dw.double() - total).abs().max().item() <= 1e-5 * total.abs().max().item()


def test_triangle_update_more_batch_items_than_grid_z_holds(device):
    """600 pair tensors of 32 x 32 x 128: the triangular contraction is a batched product over 128 * 600 = 76 800
    (channel, batch) items, more than grid.z indexes - it runs as two launches.  Every batch element must come out as in
    a call of its own."""
    from cuequivariance_amd.cuet import triangle_multiplicative_update as tmu

    B, N, D = 600, 32, 128
    dtype = torch.bfloat16
    g = torch.Generator(device=device).manual_seed(7)
    ws = {k: (torch.randn(*shape, device=device, generator=g) * 0.09).to(dtype)
          for k, shape in (("p_in_weight", (2 * D, D)), ("g_in_weight", (2 * D, D)), ("p_out_weight", (D, D)), ("g_out_weight", (D, D)))}
    x = torch.randn(B, N, N, D, device=device, generator=g).to(dtype).requires_grad_(True)
    mask = (torch.rand(B, N, N, device=device, generator=g) > 0.1).to(dtype)
    cot = torch.randn(B, N, N, D, device=device, generator=g).to(dtype)
    for direction in ("outgoing", "incoming"):
        out = tmu(x, direction, mask=mask, **ws)
        (dx,) = torch.autograd.grad(out, [x], cot)
        for b in (0, 511, 512, 599):  # 65 535 = 128 * 511 + 127: element 511 straddles the two launches
            xb = x[b:b + 1].detach().requires_grad_(True)
            ob = tmu(xb, direction, mask=mask[b:b + 1], **ws)
            (db,) = torch.autograd.grad(ob, [xb], cot[b:b + 1])
            assert torch.equal(out[b:b + 1], ob) and torch.equal(dx[b:b + 1], db), (direction, b)


def test_indexed_linear_more_rows_than_one_launch_takes(device):
    """9 500 000 rows in three weight classes (one of them empty, one of 9 499 900 rows): the rows-grouped launches take
    8.4 M rows each, so the batch runs as two row ranges with class offsets relative to each.  Against the plain Linear
    applied per class."""
    from cuequivariance_amd import cuet

    irreps = cue.Irreps("O3", "32x0e+32x1o")
    m = cuet.Linear(irreps, irreps, layout=cue.ir_mul, internal_weights=False, weight_classes=3, method="indexed_linear")
    plain = cuet.Linear(irreps, irreps, layout=cue.ir_mul, internal_weights=False, method="fused_tp")
    Z = 9_500_000
    g = torch.Generator(device=device).manual_seed(8)
    x = torch.randn(Z, irreps.dim, device=device, generator=g)
    w = torch.randn(3, m.weight_numel, device=device, generator=g)
    cot = torch.randn(Z, irreps.dim, device=device, generator=g)
    idx = torch.zeros(Z, dtype=torch.int32, device=device)
    idx[-100:] = 2
    a, b = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    out = m(a, b, weight_indices=idx)
    dx, dw = torch.autograd.grad(out, [a, b], cot)
    assert dw[1].abs().max().item() == 0
    for c, (lo, hi) in ((0, (0, Z - 100)), (2, (Z - 100, Z))):
        a2, b2 = x[lo:hi].clone().requires_grad_(True), w[c:c + 1].clone().requires_grad_(True)
        o2 = plain(a2, b2)
        dx2, dw2 = torch.autograd.grad(o2, [a2, b2], cot[lo:hi])
        # (both weight gradients are float32 sums over 9.5 million rows, accumulated in different orders)
        for name, u, v, tol in (("out", out[lo:hi], o2, 1e-5), ("dx", dx[lo:hi], dx2, 1e-5), ("dw", dw[c:c + 1], dw2, 3e-4)):
            assert (u - v).abs().max().item() <= tol * v.abs().max().item(), (name, c)
