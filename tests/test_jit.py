"""Kernels generated, compiled and loaded at first use for a channel-wise descriptor the library was not built for
(``cuequivariance_amd/jit.py``): registration on the CPU, parity against the oracle and against the table-driven kernels
on the GPU."""

import pytest
import torch

from cuequivariance_amd import cue, jit
from cuequivariance_amd.tables import U1dTables
from oracle.naive import naive_segmented_polynomial, spec_from_polynomial


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


def test_tuning_splits_descriptors_that_would_run_one_wavefront_per_simd():
    """Register estimate: the 40-channel l <= 2 product fits as it is; the l <= 3 product in float64 would be left with
    one wavefront per SIMD and is dealt out to two wavefronts with disjoint x1 segments (forward and backward)."""
    from cuequivariance_amd import jit
    from cuequivariance_amd.codegen import channelwise as cw
    from cuequivariance_amd.codegen.registry import channelwise_tables

    def structure(i1, i2, filt):
        t = channelwise_tables(i1, i2, filt)
        _, paths = t.operation(0)
        return cw.analyze(t.operand_extent, t.buffer_num_segments, [(*idx, c) for idx, c in paths])

    small = structure("40x0e+40x1o+40x2e", "0e+1o+2e", "0e+1o+2e")
    assert jit._tuning(small, "double")["fwd_split"] == 1 and jit._tuning(small, "double")["bwd_split"] == 1
    big = structure("24x0e+24x1o+24x2e+24x3o", "0e+1o+2e+3o", "0e+1o+2e+3o")
    assert jit._tuning(big, "float")["fwd_split"] == 1
    tune = jit._tuning(big, "double")
    assert tune["fwd_split"] == 2 and tune["bwd_split"] == 2 and tune["fwd_waves"] == 2 and tune["bwd_waves"] == 2
    groups = cw._split_blocks(big, 2)
    seg = [{i for blk in g for i in blk.i_list} for g in groups]
    assert len(groups) == 2 and not (seg[0] & seg[1]) and seg[0] | seg[1] == set(range(16))
    assert sorted(blk.b for g in groups for blk in g) == list(range(23))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,irreps", [(torch.float32, "40x0e+40x1o+40x2e"), (torch.float64, "40x0e+40x1o+40x2e"),
                                          (torch.float64, "24x0e+24x1o+24x2e+24x3o")])
def test_jit_kernels_match_oracle_and_generic(device, dtype, irreps, jit_on):
    """Kernels compiled at first use against the oracle; the last case is dealt out to two wavefronts per batch row
    (see the tuning test above), the others run one."""
    from cuequivariance_amd import cuet

    i1 = cue.Irreps("O3", irreps)
    lmax = 3 if "3o" in irreps else 2
    i2 = cue.Irreps("O3", "0e+1o+2e+3o" if lmax == 3 else "0e+1o+2e")
    filt = ["0e", "1o", "2e", "3o"][: lmax + 1]
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


@pytest.mark.gpu
def test_general_generator_second_derivative_and_harmonics(device, jit_on):
    """Plans outside the two generated families get a unit of their own from the general generator: the backward of the
    backward of a channel-wise product (double backward against the CPU oracle's autograd) and spherical harmonics (a plan
    without channel mode: a lane per row)."""
    from cuequivariance_amd import cuet

    i1, i2 = cue.Irreps("O3", "24x0e+24x1o"), cue.Irreps("O3", "0e+1o")
    m = cuet.ChannelWiseTensorProduct(i1, i2, ["0e", "1o"], layout=cue.ir_mul, shared_weights=False, internal_weights=False,
                                      device=device, dtype=torch.float64)
    g = torch.Generator().manual_seed(9)
    N, Z = 13, 90
    x1 = torch.randn(N, i1.dim, generator=g, dtype=torch.float64)
    x2 = torch.randn(Z, i2.dim, generator=g, dtype=torch.float64)
    w = torch.randn(Z, m.weight_numel, generator=g, dtype=torch.float64)
    snd = torch.randint(0, N, (Z,), generator=g, dtype=torch.int32)
    rcv = torch.sort(torch.randint(0, N, (Z,), generator=g, dtype=torch.int32))[0]
    cot = torch.randn(N, m.irreps_out.dim, generator=g, dtype=torch.float64)
    v = torch.randn(Z, i2.dim, generator=g, dtype=torch.float64)

    def second(w_, x1_, x2_, fwd):
        out = fwd(w_, x1_, x2_)
        (gx2,) = torch.autograd.grad(out, [x2_], cot.to(out.device), create_graph=True)
        return torch.autograd.grad((gx2 * v.to(out.device)).sum(), [w_, x1_, x2_], allow_unused=True)

    spec = spec_from_polynomial(m.f._polynomial_orig)
    a = [t.clone().requires_grad_(True) for t in (w, x1, x2)]
    want = second(*a, lambda w_, x1_, x2_: naive_segmented_polynomial(spec, [w_, x1_, x2_], {1: snd}, {0: N}, {0: rcv})[0])
    b = [t.clone().to(device).requires_grad_(True) for t in (w, x1, x2)]
    got = second(*b, lambda w_, x1_, x2_: m(x1_, x2_, w_, indices_1=snd.to(device), indices_out=rcv.to(device), size_out=N))
    for p, q in zip(want, got):
        if p is None:
            assert q is None or q.abs().max().item() == 0
        else:
            assert (q.cpu() - p).abs().max().item() <= 1e-12 * max(p.abs().max().item(), 1e-30)
    plan = m.f.m._plan(torch.float64)
    assert plan.specialised(device)

    sh = cuet.SphericalHarmonics([0, 1, 2, 3], normalize=False, device=device)
    vec = torch.randn(1000, 3, generator=g, dtype=torch.float64)
    y = sh(vec.to(device))
    assert sh.f.m._plan(torch.float64).specialised(device)
    # closed forms: Y_0 = 1, Y_1 = sqrt(3) x, and sum_m Y_lm^2 = (2 l + 1) |x|^(2 l) (component normalisation)
    r2 = (vec * vec).sum(1)
    assert torch.allclose(y[:, 0].cpu(), torch.ones(1000, dtype=torch.float64), atol=1e-12)
    assert torch.allclose(y[:, 1:4].cpu(), 3 ** 0.5 * vec, atol=1e-12)
    for l, lo in ((2, 4), (3, 9)):
        assert torch.allclose((y[:, lo:lo + 2 * l + 1].cpu() ** 2).sum(1), (2 * l + 1) * r2 ** l, rtol=1e-11)


def _dense_of(module):
    return next(x for x in module.modules() if type(x).__name__ == "SegmentedPolynomialDense")


def test_fully_connected_generator_limits():
    """What the fused fully connected generator takes: multiplicities that are multiples of 32 up to 128, rows of at most
    256 columns; the source it emits holds the three kernels and their C entry points."""
    from cuequivariance_amd import cuet
    from cuequivariance_amd.codegen import fullyconnected as fc

    def dense(i1, i2, i3):
        return _dense_of(cuet.FullyConnectedTensorProduct(cue.Irreps("O3", i1), cue.Irreps("O3", i2), cue.Irreps("O3", i3),
                                                          layout=cue.ir_mul, internal_weights=False))

    d = dense("64x0e+64x1o", "0e+1o+2e", "64x0e+64x1o")
    assert fc.supported(d.paths, 9, 256, 256, 4) and fc.supported(d.paths, 9, 256, 256, 2)
    src = fc.emit_unit(d.paths, 9, 256, 256, "float")
    for name in ("fwd_kernel", "dx1_kernel", "dx2_kernel", "dx12_kernel", "dw_kernel"):
        assert name in src
    # both input gradients in one pass: float objects with multiplicities that are multiples of 64 only
    assert fc.dx12_supported(d.paths, 256)
    assert "dx12_kernel" not in fc.emit_unit(d.paths, 9, 256, 256, "uint16_t")
    mixed = dense("32x0e+64x1o", "0e+1o", "96x0e+32x1o")
    assert not fc.dx12_supported(mixed.paths, mixed.input_sizes[1])
    assert "return -2;" in fc.emit_unit(mixed.paths, mixed.input_sizes[2], mixed.input_sizes[1], mixed.out_size, "float")
    # every entry point the header of the generated objects declares is defined, with the declared number of arguments
    import pathlib
    import re

    header = (pathlib.Path(__file__).resolve().parent.parent / "include" / "cueq_amd_generated.h").read_text()
    declared = re.findall(r"^int (fcj_\w+)\(([^;]*)\);", header, flags=re.M | re.S)
    assert {n for n, _ in declared} == {"fcj_fwd", "fcj_dx1", "fcj_dx2", "fcj_dx12", "fcj_dw_blocks", "fcj_dw"}
    for name, args in declared:
        m = re.search(r'extern "C" int %s\(([^)]*)\)' % name, src)
        assert m, name
        assert len(m.group(1).split(",")) == len(args.split(",")), name
    d = dense("8x0e+3x1o", "0e+1o", "5x0e+7x1o")
    assert not fc.supported(d.paths, 4, d.input_sizes[1], d.out_size, 4)
    d = dense("128x0e+128x1o", "0e+1o", "128x0e+128x1o")  # 512 columns a row
    assert not fc.supported(d.paths, 4, d.input_sizes[1], d.out_size, 4)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("i1,i2,i3,Z", [
    ("64x0e+64x1o", "0e+1o+2e", "64x0e+64x1o", 777),   # ragged: the last 32-row tile holds 9 rows
    ("32x0e+64x1o", "0e+1o", "96x0e+32x1o", 2500),     # mixed block shapes, a wavefront walks more than one tile on few CUs
    ("32x0e", "0e+1o", "32x1o", 1),
    ("128x0e+64x0e", "0e+1o", "64x0e+64x1o", 333),     # a segment of 128 channels: two tiles per half in the one-pass input gradients
])
def test_fused_fully_connected_matches_oracle_and_tables(device, dtype, i1, i2, i3, Z, jit_on):
    """The generated fully connected kernels (weights resident in LDS, products scaled in registers) against the CPU
    oracle, and against the table-driven GEMM path of the same module at the same tolerance."""
    from cuequivariance_amd import cuet

    m = cuet.FullyConnectedTensorProduct(cue.Irreps("O3", i1), cue.Irreps("O3", i2), cue.Irreps("O3", i3), layout=cue.ir_mul,
                                         internal_weights=False)
    g = torch.Generator().manual_seed(Z)
    ins = [torch.randn(1, m.weight_numel, dtype=torch.float64, generator=g),
           torch.randn(Z, m.irreps_in1.dim, dtype=torch.float64, generator=g),
           torch.randn(Z, m.irreps_in2.dim, dtype=torch.float64, generator=g)]
    rounded = [t.to(dtype).double() for t in ins]
    spec = spec_from_polynomial(m.f._polynomial_orig)
    a = [t.clone().requires_grad_(True) for t in rounded]
    ref = naive_segmented_polynomial(spec, a)[0]
    cot = torch.randn(ref.shape, dtype=torch.float64, generator=g).to(dtype).double()
    want = (ref,) + torch.autograd.grad(ref, a, cot)

    def run():
        b = [t.to(dtype).to(device).requires_grad_(True) for t in rounded]
        out = m.f(b)[0]
        return (out,) + torch.autograd.grad(out, b, cot.to(dtype).to(device))

    got = run()
    d = _dense_of(m)
    assert d._fused.get((dtype, True)) is not None, "the generated kernels were not built"
    jit.enable(False)
    tables = run()
    assert d._fused.get((dtype, False)) is None  # (half: computed in float32 by the table-driven kernels, rounded once)
    tol = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-3}[dtype]
    for name, u, v, t in zip(("out", "dw", "dx1", "dx2"), got, want, tables):
        assert u.dtype == dtype and u.shape == v.shape
        scale = max(v.abs().max().item(), 1e-30)
        assert (u.double().cpu() - v).abs().max().item() <= tol * scale, name
        assert (u.double() - t.double()).abs().max().item() <= 2 * tol * scale, name + " vs tables"


@pytest.mark.gpu
@pytest.mark.parametrize("on", [True, False])
def test_fully_connected_unaligned_rows(device, jit_on, on):
    """The fully connected kernels (generated and table-driven) move rows in 16-byte pieces; an operand view that starts
    4 bytes off such a boundary is copied to aligned storage first and gives what an aligned copy gives."""
    from cuequivariance_amd import cuet

    jit.enable(on)
    m = cuet.FullyConnectedTensorProduct(cue.Irreps("O3", "32x0e+32x1o"), cue.Irreps("O3", "0e+1o"), cue.Irreps("O3", "32x0e+32x1o"),
                                         layout=cue.ir_mul, internal_weights=False)
    g = torch.Generator().manual_seed(3)
    Z = 100
    w = torch.randn(1, m.weight_numel, generator=g).to(device)
    x2 = torch.randn(Z, 4, generator=g).to(device)
    flat = torch.randn(1 + Z * 128, generator=g).to(device)
    x1_off = flat[1:].view(Z, 128)            # contiguous rows, first element 4 bytes past a 16-byte boundary
    x1_al = x1_off.clone()
    cot_off = torch.randn(1 + Z * 128, generator=g).to(device)[1:].view(Z, 128)
    assert x1_off.data_ptr() % 16 == 4 and x1_al.data_ptr() % 16 == 0 and cot_off.data_ptr() % 16 == 4
    d = _dense_of(m)
    assert d.fused_unit(torch.float32, x1_off) is None

    def run(x1, cot):
        a = [w.clone().requires_grad_(True), x1.detach().requires_grad_(True), x2.clone().requires_grad_(True)]
        out = m.f(a)[0]
        return (out,) + torch.autograd.grad(out, a, cot)

    want = run(x1_al, cot_off.clone())
    got = run(x1_off, cot_off)
    assert (d._fused.get((torch.float32, True)) is not None) == on
    for u, v in zip(got, want):
        assert torch.equal(u, v)


@pytest.mark.gpu
def test_fused_fully_connected_rows_beyond_2g_elements(device, jit_on):
    """9 000 000 rows of 256 columns (2.3e9 elements per operand) through the generated kernels: one call against the
    same rows in two halves (per-row results do not depend on the batch they are computed in; weight gradients add)."""
    import gc

    from cuequivariance_amd import cuet

    i1, i2 = cue.Irreps("O3", "64x0e+64x1o"), cue.Irreps("O3", "0e+1o+2e")
    m = cuet.FullyConnectedTensorProduct(i1, i2, i1, layout=cue.ir_mul, internal_weights=False)
    Z = 9_000_000
    assert Z * i1.dim > 2 ** 31
    g = torch.Generator(device=device).manual_seed(4)
    x1 = torch.randn(Z, i1.dim, device=device, generator=g)
    x2 = torch.randn(Z, i2.dim, device=device, generator=g)
    w = torch.randn(1, m.weight_numel, device=device, generator=g)
    cot = torch.randn(Z, i1.dim, device=device, generator=g)

    def run(lo, hi):
        a = [x1[lo:hi].requires_grad_(True), x2[lo:hi].requires_grad_(True), w.clone().requires_grad_(True)]
        out = m(a[0], a[1], a[2])
        return (out.detach(),) + torch.autograd.grad(out, a, cot[lo:hi])

    out, dx1, dx2, dw = run(0, Z)
    assert _dense_of(m)._fused.get((torch.float32, True)) is not None
    h = Z // 2
    halves = torch.zeros_like(dw, dtype=torch.float64)
    for lo, hi in ((0, h), (h, Z)):
        o, d1, d2, dwh = run(lo, hi)
        assert torch.equal(out[lo:hi], o) and torch.equal(dx1[lo:hi], d1) and torch.equal(dx2[lo:hi], d2)
        halves += dwh.double()
        del o, d1, d2, dwh
    assert (dw.double() - halves).abs().max().item() <= 1e-5 * halves.abs().max().item()  # (the halves sum in another order)
    del out, dx1, dx2, x1, x2, cot
    gc.collect()
    torch.cuda.empty_cache()


@pytest.mark.gpu
def test_fused_fully_connected_second_derivatives(device, jit_on):
    """Second derivatives through the generated fully connected kernels (each gradient is one of them again)."""
    from tests.test_gpu_dense import fc_second_derivatives

    err, m = fc_second_derivatives(device, torch.float32, "32x0e+32x1o")
    assert _dense_of(m)._fused.get((torch.float32, True)) is not None
    assert err <= 2e-5, err


@pytest.mark.gpu
@pytest.mark.parametrize("on", [False, True])
def test_scalar_output_mixing_contracting_and_scalar_paths(device, jit_on, on):
    """One scalar output fed by a path that contracts the channel mode (x[u] gy[u] -> dw[]) and by a path of scalars only
    (s[] gt[] -> dw[]) - what the weight gradient of ``w[] x[u] -> y[u]`` plus ``w[] s[] -> t[]`` looks like.  The scalar
    path must be counted once, not once per channel.  Table-driven kernels (``on`` False) and the general generator
    (True) against the oracle and against the closed form."""
    import numpy as np

    from cuequivariance_amd.cuet.uniform_1d import Uniform1dPlan, run_plan
    from cuequivariance_amd import _lib

    jit.enable(on)
    E, Z = 48, 37
    # buffers: 0 x[u] (2 segments), 1 gy[u] (2), 2 s[] (2), 3 gt[] (2) | 4 dw[] (2 scalar segments)
    tables = U1dTables.make(
        E, 4, 1, [1, 1, 0, 0, 0], [2, 2, 2, 2, 2], [0, 1, 2, 3, -1], [3, 3], [0, 1, 4, 2, 3, 4], [3, 2], [0, 9], [0, 3],
        [0, 0, 0, 1, 1, 1, 0, 1, 1,  0, 0, 0, 1, 0, 1], [2.0, -1.5, 0.5, 3.0, 0.25])
    spec = dict(
        num_inputs=4, num_outputs=1, sizes=[2 * E, 2 * E, 2, 2, 2],
        operations=[
            dict(buffers=[0, 1, 4], operand_subscripts=["u", "u", ""], coefficient_subscripts="",
                 segments=[[(E,), (E,)], [(E,), (E,)], [(), ()]], path_indices=[(0, 0, 0), (1, 1, 1), (0, 1, 1)],
                 path_coefficients=[np.array(2.0), np.array(-1.5), np.array(0.5)]),
            dict(buffers=[2, 3, 4], operand_subscripts=["", "", ""], coefficient_subscripts="",
                 segments=[[(), ()], [(), ()], [(), ()]], path_indices=[(0, 0, 0), (1, 0, 1)],
                 path_coefficients=[np.array(3.0), np.array(0.25)]),
        ])
    g = torch.Generator().manual_seed(3)
    x, gy = (torch.randn(Z, 2 * E, generator=g, dtype=torch.float64) for _ in range(2))
    sc, gt = (torch.randn(Z, 2, generator=g, dtype=torch.float64) for _ in range(2))
    want = naive_segmented_polynomial(spec, [x, gy, sc, gt])[0]
    closed = torch.stack([
        2.0 * (x[:, :E] * gy[:, :E]).sum(1) + 3.0 * sc[:, 0] * gt[:, 0],
        -1.5 * (x[:, E:] * gy[:, E:]).sum(1) + 0.5 * (x[:, :E] * gy[:, E:]).sum(1) + 0.25 * sc[:, 1] * gt[:, 0]], 1)
    assert (want - closed).abs().max().item() <= 1e-12 * closed.abs().max().item()
    plan = Uniform1dPlan(tables, torch.float64, name="mixed_scalar_output")
    B = _lib.BATCH_DIM_BATCHED
    got = run_plan(plan, [B] * 5, [-1] * 5, Z, 0, [v.to(device) for v in (x, gy, sc, gt)])[0]
    assert plan.specialised(device) == on
    assert (got.cpu() - want).abs().max().item() <= 1e-12 * want.abs().max().item()
