"""Operands in the mul_ir layout addressed by the uniform-1d kernels themselves (no transposition pass).

The reference transposes mul_ir operands to ir_mul before the product and back after it
(``cuequivariance_torch/operations/tp_channel_wise.py:118-133, 167-196``, ``primitives/transpose.py:26-83``); here the
flattened tables carry, per buffer, groups of segments stored channel-major, and every kernel family addresses rows
through them.  The checks: the addressing formula against the layout's definition (numpy reshapes), the table hash
agreeing between Python and C with layouts, and on the GPU the mul_ir module against the oracle (which works in ir_mul)
with operands and results converted by plain reshapes - forward, the three gradients, second derivatives - for the
generated, the generated-at-first-use and the table-driven kernels.
"""

import ctypes

import numpy as np
import pytest
import torch

from cuequivariance_amd import _lib, cue
from cuequivariance_amd.tables import U1dTables

TOL = {torch.float64: 1e-12, torch.float32: 1e-5}


def to_mul_ir(x: torch.Tensor, irreps) -> torch.Tensor:
    """ir_mul rows -> mul_ir rows by reshapes alone: block (ir.dim, mul) becomes (mul, ir.dim)."""
    outs, off = [], 0
    for mul, ir in irreps:
        outs.append(x[:, off: off + mul * ir.dim].reshape(-1, ir.dim, mul).transpose(1, 2).reshape(x.shape[0], -1))
        off += mul * ir.dim
    return torch.cat(outs, 1)


def channelwise_tables(ir1="32x0e+32x1o+32x2e", ir2="0e+1o+2e", filt="0e+1o+2e"):
    e = cue.descriptors.channelwise_tensor_product(cue.Irreps("O3", ir1), cue.Irreps("O3", ir2), filt)
    t = U1dTables.from_polynomial(e.polynomial.flatten_coefficient_modes().squeeze_modes())
    groups = {1: [ir.dim for _, ir in e.inputs[1].irreps], 3: [ir.dim for _, ir in e.outputs[0].irreps]}
    return e, t, groups


# --------------------------------------------------------------------------- host side
def test_segment_addressing_is_the_mul_ir_layout():
    e, t, groups = channelwise_tables()
    tl = t.with_layouts(groups)
    E = t.operand_extent
    for b, irreps in ((1, e.inputs[1].irreps), (3, e.outputs[0].irreps)):
        width = t.width(b)
        row = torch.arange(width, dtype=torch.float64).reshape(1, width)  # ir_mul row: element id = seg * E + u
        row_mul_ir = to_mul_ir(row, irreps)[0].numpy()
        addr = tl.segment_addressing(b)
        assert len(addr) == t.buffer_num_segments[b]
        for seg, (base, stride) in enumerate(addr):
            got = row_mul_ir[base + stride * np.arange(E)]
            assert np.array_equal(got, seg * E + np.arange(E)), (b, seg)
    # buffers without a layout keep segment-major addressing
    assert tl.segment_addressing(0) == [(s * E, 1) for s in range(t.buffer_num_segments[0])]


def test_layouts_follow_the_operands_through_the_backward_tables():
    _, t, groups = channelwise_tables()
    tb = t.with_layouts(groups).backward((True, True, True))
    # inputs w, x1, x2, cotangent of out; outputs dw, dx1, dx2
    assert [tuple(tb.layout(b)) for b in range(7)] == [(), tuple(groups[1]), (), tuple(groups[3]), (), tuple(groups[1]), ()]
    only_x1 = t.with_layouts(groups).backward((False, True, False))
    assert tuple(only_x1.layout(3)) == tuple(groups[3]) and tuple(only_x1.layout(4)) == tuple(groups[1])


def test_groups_must_partition_the_segments():
    _, t, groups = channelwise_tables()
    with pytest.raises(ValueError):
        t.with_layouts({1: [1, 3]})
    with pytest.raises(ValueError):
        t.with_layouts({2: [1, 3, 5]})  # x2 carries no channel
    assert t.with_layouts({1: [1] * 9}).layouts == ()  # groups of one segment: the default layout


@pytest.mark.parametrize("math_code", [0, 1])
def test_table_hash_with_layouts_agrees_between_python_and_c(math_code):
    lib = _lib.load()
    _, t, groups = channelwise_tables()
    tl = t.with_layouts(groups)
    seen = set()
    for tables in (t, tl, t.with_layouts({1: groups[1]}), t.with_layouts({3: groups[3]}), tl.backward((True, True, True))):
        desc, keep = _lib.make_desc(tables, math_code)
        h = ctypes.c_uint64()
        has_spec = lib.cueq_u1d_desc_info(ctypes.byref(desc), ctypes.byref(h))
        assert h.value == tables.content_hash(math_code)
        seen.add(h.value)
        # generated at build time: both layouts of x1 and the output together, not the mixed ones
        assert has_spec == (0 if tables.layouts and (not tables.layout(1) or not tables.layout(3)) else 1)
    assert len(seen) == 5


@pytest.mark.parametrize("math_code", [0, 1])
def test_groups_of_one_segment_hash_as_the_default_rows(math_code):
    """A descriptor handed to the C ABI with every group of a buffer one segment long describes the default rows: its hash
    (and with it the generated kernels it finds) is that of the descriptor without a layout."""
    lib = _lib.load()
    _, t, groups = channelwise_tables()
    plain, keep0 = _lib.make_desc(t, math_code)
    want = ctypes.c_uint64()
    has_plain = lib.cueq_u1d_desc_info(ctypes.byref(plain), ctypes.byref(want))
    nbuf = t.num_inputs + t.num_outputs
    # spelled out by hand: buffers 1 and 3 in groups of one, then buffer 1 in groups of one next to a real layout of buffer 3
    for lay in ({1: [1] * t.buffer_num_segments[1], 3: [1] * t.buffer_num_segments[3]}, {1: [1] * t.buffer_num_segments[1], 3: list(groups[3])}):
        desc, keep = _lib.make_desc(t, math_code)
        n = _lib.int32_array([len(lay.get(b, ())) for b in range(nbuf)])
        d = _lib.int32_array([x for b in range(nbuf) for x in lay.get(b, ())])
        desc.layout_num_groups, desc.layout_group_dims = n, d
        got = ctypes.c_uint64()
        has = lib.cueq_u1d_desc_info(ctypes.byref(desc), ctypes.byref(got))
        same = t.with_layouts(lay)
        assert got.value == same.content_hash(math_code)
        if not same.layouts:
            assert got.value == want.value and has == has_plain == 1


def test_channelwise_module_drops_its_transpositions():
    from cuequivariance_amd import cuet

    ir1, ir2 = cue.Irreps("O3", "32x0e+32x1o+32x2e"), cue.Irreps("O3", "0e+1o+2e")
    m = cuet.ChannelWiseTensorProduct(ir1, ir2, "0e+1o+2e", layout=cue.mul_ir, shared_weights=False)
    assert isinstance(m.transpose_in1.f, torch.nn.Identity) and isinstance(m.transpose_out.f, torch.nn.Identity)
    assert tuple(m.f.m.tables.layout(1)) == (1, 3, 5) and len(m.f.m.tables.layout(3)) == len(m.irreps_out)
    m = cuet.ChannelWiseTensorProduct(ir1, ir2, "0e+1o+2e", layout=cue.ir_mul, shared_weights=False)
    assert m.f.m.tables.layouts == ()
    # a mixed request: only the operand that is mul_ir gets a layout
    m = cuet.ChannelWiseTensorProduct(ir1, ir2, "0e+1o+2e", layout=cue.ir_mul, layout_out=cue.mul_ir, shared_weights=False)
    assert not m.f.m.tables.layout(1) and m.f.m.tables.layout(3)


# --------------------------------------------------------------------------- GPU parity
def assert_close(got, ref, tol, what):
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    got, ref = got.detach().cpu().double(), ref.detach().cpu().double()
    scale = max(ref.abs().max().item(), 1e-30)
    err = (got - ref).abs().max().item()
    assert err <= tol * scale, f"{what}: max err {err:.3e} > {tol:.0e} * {scale:.3e}"


def run_case(device, ir1, ir2, filt, N, Z, dtype, seed, indexed=True, layout_in1=cue.mul_ir, layout_out=cue.mul_ir):
    """mul_ir module against the oracle (ir_mul) with reshaped operands; returns the module."""
    from cuequivariance_amd import cuet
    from oracle.naive import naive_segmented_polynomial, spec_from_polynomial

    irreps1, irreps2 = cue.Irreps("O3", ir1), cue.Irreps("O3", ir2)
    m = cuet.ChannelWiseTensorProduct(irreps1, irreps2, filt, layout=cue.ir_mul, layout_in1=layout_in1, layout_out=layout_out,
                                      shared_weights=False)
    conv1 = (lambda x: to_mul_ir(x, irreps1)) if layout_in1 == cue.mul_ir else (lambda x: x)
    conv3 = (lambda x: to_mul_ir(x, m.irreps_out)) if layout_out == cue.mul_ir else (lambda x: x)
    spec = spec_from_polynomial(m.f._polynomial_orig)
    g = torch.Generator().manual_seed(seed)
    rows1 = N if indexed else Z
    x1 = torch.randn(rows1, irreps1.dim, dtype=torch.float64, generator=g).to(dtype)
    x2 = torch.randn(Z, irreps2.dim, dtype=torch.float64, generator=g).to(dtype)
    w = torch.randn(Z, m.weight_numel, dtype=torch.float64, generator=g).to(dtype)
    snd = torch.randint(0, max(N, 1), (Z,), generator=g, dtype=torch.int32)
    rcv = torch.sort(torch.randint(0, max(N, 1), (Z,), generator=g, dtype=torch.int32))[0]
    cot = torch.randn(N if indexed else Z, m.irreps_out.dim, dtype=torch.float64, generator=g).to(dtype)
    a = [t.clone().requires_grad_(True) for t in (w, x1, x2)]
    if indexed:
        ref = naive_segmented_polynomial(spec, a, {1: snd}, {0: N}, {0: rcv})[0]
    else:
        ref = naive_segmented_polynomial(spec, a)[0]
    ref_grads = torch.autograd.grad((ref * cot).sum(), a)
    b = [t.to(device).requires_grad_(True) for t in (w, conv1(x1), x2)]
    if indexed:
        out = m(b[1], b[2], b[0], indices_1=snd.to(device), indices_out=rcv.to(device), size_out=N)
    else:
        out = m(b[1], b[2], b[0])
    grads = torch.autograd.grad(out, b, conv3(cot).to(device))
    tol = TOL[dtype]
    assert_close(out, conv3(ref), tol, "out")
    assert_close(grads[0], ref_grads[0], tol, "dw")
    assert_close(grads[1], conv1(ref_grads[1]), tol, "dx1")
    assert_close(grads[2], ref_grads[2], tol, "dx2")
    return m


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("deterministic", ["0", "1"])
def test_cfg2_descriptor_mul_ir(device, dtype, deterministic, monkeypatch):
    """128 channels, l <= 3, 300 nodes / 4000 edges, gathered x1 and scattered output, both dx1 scatter policies: the
    kernels generated at build time for the mul_ir layout."""
    monkeypatch.setenv("CUEQ_DETERMINISTIC", deterministic)
    m = run_case(device, "128x0e+128x1o+128x2e+128x3o", "0e+1o+2e+3o", "0e+1o+2e+3o", 300, 4000, dtype, seed=11)
    plan = m.f.m._plan(dtype)
    assert plan.specialised(device) and plan.backward_plan((True, True, True)).specialised(device)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_cfg1_descriptor_mul_ir_batched(device, dtype):
    m = run_case(device, "32x0e+32x1o+32x2e", "0e+1o+2e", "0e+1o+2e", 0, 1000, dtype, seed=12, indexed=False)
    assert m.f.m._plan(dtype).specialised(device)


@pytest.mark.gpu
@pytest.mark.parametrize("forced_generic", ["", "1"])
def test_other_descriptor_mul_ir(device, forced_generic, monkeypatch):
    """48 channels (not a multiple of the wavefront), a filter that drops irreps: kernels generated at first use, or
    (forced) the table-driven kernels."""
    if forced_generic:
        monkeypatch.setenv("CUEQ_FORCE_GENERIC", "1")
    for dtype in (torch.float64, torch.float32):
        run_case(device, "48x0e+48x1o+48x1e", "0e+1o+2e", "0e+1o+1e+2o", 40, 333, dtype, seed=13)


@pytest.mark.gpu
@pytest.mark.parametrize("which", ["in1", "out"])
def test_one_operand_mul_ir(device, which):
    """Only x1, or only the output, in mul_ir: descriptors the build holds no kernels for."""
    kw = dict(layout_in1=cue.mul_ir, layout_out=cue.ir_mul) if which == "in1" else dict(layout_in1=cue.ir_mul, layout_out=cue.mul_ir)
    run_case(device, "32x0e+32x1o+32x2e", "0e+1o+2e", "0e+1o+2e", 50, 400, torch.float64, seed=14, **kw)


@pytest.mark.gpu
def test_second_derivative_mul_ir(device):
    """Second-order gradients (the double backward runs units of the general generator, or the table-driven kernels,
    on tables whose buffers keep their layouts)."""
    from cuequivariance_amd import cuet
    from oracle.naive import naive_segmented_polynomial, spec_from_polynomial

    irreps1, irreps2 = cue.Irreps("O3", "16x0e+16x1o"), cue.Irreps("O3", "0e+1o")
    m = cuet.ChannelWiseTensorProduct(irreps1, irreps2, "0e+1o", layout=cue.mul_ir, shared_weights=False)
    spec = spec_from_polynomial(m.f._polynomial_orig)
    g = torch.Generator().manual_seed(15)
    Z, R = 23, 7
    w = torch.randn(Z, m.weight_numel, dtype=torch.float64, generator=g)
    x1 = torch.randn(R, irreps1.dim, dtype=torch.float64, generator=g)
    x2 = torch.randn(Z, irreps2.dim, dtype=torch.float64, generator=g)
    snd = torch.randint(0, R, (Z,), generator=g, dtype=torch.int32)
    rcv = torch.randint(0, R, (Z,), generator=g, dtype=torch.int32)

    def scalar(fn, ins):
        out = fn(ins)
        gs = torch.autograd.grad(out.square().sum(), ins, create_graph=True)
        return sum(gi.sin().sum() for gi in gs)

    a = [t.clone().requires_grad_(True) for t in (w, x1, x2)]
    ra = scalar(lambda ins: naive_segmented_polynomial(spec, ins, {1: snd}, {0: R}, {0: rcv})[0], a)
    ga = torch.autograd.grad(ra, a)
    # sin() of the first-order gradients is applied elementwise, so the layout of dx1 does not change the scalar
    b = [t.to(device).requires_grad_(True) for t in (w, to_mul_ir(x1, irreps1), x2)]
    rb = scalar(lambda ins: m(ins[1], ins[2], ins[0], indices_1=snd.to(device), indices_out=rcv.to(device), size_out=R), b)
    gb = torch.autograd.grad(rb, b)
    assert_close(rb.reshape(1), ra.reshape(1), 1e-12, "scalar")
    assert_close(gb[0], ga[0], 1e-11, "second-order dw")
    assert_close(gb[1], to_mul_ir(ga[1], irreps1), 1e-11, "second-order dx1")
    assert_close(gb[2], ga[2], 1e-11, "second-order dx2")


# --------------------------------------------------------------------------- kernels generated at first use
@pytest.mark.gpu
@pytest.mark.parametrize("dtype,ir1,lmax", [(torch.float32, "40x0e+40x1o+40x2e", 2), (torch.float64, "24x0e+24x1o+24x2e+24x3o", 3)])
def test_first_use_kernels_mul_ir(device, dtype, ir1, lmax, jit_on):
    """Channel-wise units compiled at first use for mul_ir operands (the second case is dealt out to two wavefronts per
    batch row), forward and the fused backward."""
    ir2 = "0e+1o+2e+3o" if lmax == 3 else "0e+1o+2e"
    m = run_case(device, ir1, ir2, ir2, 31, 500, dtype, seed=16)
    plan = m.f.m._plan(dtype)
    assert plan.specialised(device) and plan.backward_plan((True, True, True)).specialised(device)


@pytest.mark.gpu
def test_first_use_general_units_mul_ir(device, jit_on):
    """Second derivatives with compilation at first use on: units of the general generator on tables with layouts."""
    test_second_derivative_mul_ir(device)


# --------------------------------------------------------------------------- symmetric contraction
def run_symmetric_case(device, irreps_in, irreps_out, degree, nel, Z, dtype, seed):
    """``SymmetricContraction(layout=mul_ir)`` (x and the output addressed in place) against the oracle in ir_mul."""
    from cuequivariance_amd import cuet
    from oracle.naive import naive_segmented_polynomial, spec_from_polynomial

    m = cuet.SymmetricContraction(cue.Irreps("O3", irreps_in), cue.Irreps("O3", irreps_out), degree, nel, layout=cue.mul_ir,
                                  dtype=dtype, device=device)
    assert isinstance(m.transpose_in.f, torch.nn.Identity) and isinstance(m.transpose_out.f, torch.nn.Identity)
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(Z, m.irreps_in.dim, dtype=torch.float64, generator=gen).to(dtype)
    idx = torch.randint(0, nel, (Z,), generator=gen, dtype=torch.int32)
    w = m.weight.detach().cpu().clone()
    a = [w.flatten(1).double().requires_grad_(True), x.double().requires_grad_(True)]
    ref = naive_segmented_polynomial(spec_from_polynomial(m.etp.polynomial), a, {0: idx})[0]
    cot = torch.randn(ref.shape, dtype=torch.float64, generator=gen).to(dtype)
    ref_dw, ref_dx = torch.autograd.grad(ref, a, cot.double())
    xg = to_mul_ir(x, m.irreps_in).to(device).requires_grad_(True)
    out = m(xg, idx.to(device))
    dw, dx = torch.autograd.grad(out, [m.weight, xg], to_mul_ir(cot, m.irreps_out).to(device))
    tol = TOL[dtype]
    assert_close(out, to_mul_ir(ref, m.irreps_out), tol, "out")
    assert_close(dw.flatten(1), ref_dw, tol, "dw")
    assert_close(dx, to_mul_ir(ref_dx, m.irreps_in), tol, "dx")
    return m


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_symmetric_contraction_cfg3_descriptor_mul_ir(device, dtype):
    """128 channels, 0e+1o+2e+3o -> 0e+1o, degree 3, 10 element types, 40 nodes: the build's mul_ir unit."""
    m = run_symmetric_case(device, "128x0e+128x1o+128x2e+128x3o", "128x0e+128x1o", 3, 10, 40, dtype, seed=31)
    plan = m.f.m._plan(dtype)
    assert plan.specialised(device) and plan.backward_plan((True, True)).specialised(device)
    assert tuple(plan.tables.layout(1)) == (1, 3, 5, 7) and tuple(plan.tables.layout(2)) == (1, 3)


@pytest.mark.gpu
@pytest.mark.parametrize("first_use", [False, True])
def test_symmetric_contraction_other_descriptor_mul_ir(device, first_use, tmp_path, monkeypatch):
    """48 channels, degree 2: the table-driven kernels, and a unit compiled at first use."""
    from cuequivariance_amd import jit

    was = jit.enabled()
    if first_use:
        monkeypatch.setenv("CUEQ_AMD_JIT_CACHE", str(tmp_path))
    jit.enable(first_use)
    try:
        m = run_symmetric_case(device, "48x0e+48x1o+48x2e", "48x0e+48x1o", 2, 3, 77, torch.float64, seed=32)
        assert m.f.m._plan(torch.float64).specialised(device) == first_use
    finally:
        jit.enable(was)
