"""Fully connected tensor product with a weight row per batch row (the product inside the reference's
``FullyConnectedTensorProductConv``, ``cuequivariance_torch/layers/tp_conv_fully_connected.py:216-276``): the kernels of
``cuequivariance_amd/codegen/fullyconnected_rows.py`` against the oracle - forward and the three gradients from the fused
backward, plain batch and gather / scatter by index, both policies for the gathered operand's gradient."""

import pytest
import torch

from cuequivariance_amd import cue, jit
from cuequivariance_amd.codegen import fullyconnected_rows as fcr
from cuequivariance_amd.cue import descriptors
from cuequivariance_amd.tables import U1dTables


def flattened_tables(polynomial):
    from cuequivariance_amd.codegen.registry import flattened_fully_connected_tables

    return flattened_fully_connected_tables(polynomial)


def test_structure_of_the_descriptor():
    i1, i2 = cue.Irreps("O3", "64x0e+64x1o"), cue.Irreps("O3", "0e+1o+2e")
    e = descriptors.fully_connected_tensor_product(i1, i2, i1)
    st = fcr.analyze(e.polynomial)
    assert (st.U, st.Wd, st.width_w, st.width_x1, st.width_x2, st.width_out) == (64, 64, 20480, 256, 9, 256)
    # 0e0e0e, 0e1o1o, 1o0e1o, 1o1o0e, 1o2e1o: non-zeros of the Clebsch-Gordan tensors
    assert [len(b.entries) for b in st.blocks] == [1, 3, 3, 3, 11]
    assert [b.w_off for b in st.blocks] == [4096 * n for n in range(5)]
    t = flattened_tables(e.polynomial)
    assert jit.is_row_weight_fully_connected(t, e.polynomial)
    assert jit._family(t, None, e.polynomial) == "fc_rows" and jit.has_fused_backward(t, None, e.polynomial)
    # not this family: different multiplicities in one operand, a second operand with multiplicity, a channel-wise product
    assert fcr.analyze(descriptors.fully_connected_tensor_product(cue.Irreps("O3", "8x0e+4x1o"), i2, i1).polynomial) is None
    assert fcr.analyze(descriptors.fully_connected_tensor_product(i1, cue.Irreps("O3", "2x0e"), i1).polynomial) is None
    assert fcr.analyze(descriptors.channelwise_tensor_product(i1, i2, "0e+1o").polynomial) is None
    assert fcr.analyze(descriptors.fully_connected_tensor_product(cue.Irreps("O3", "128x0e"), i2, i1).polynomial) is None


def test_unit_compiles_and_registers_under_both_hashes(jit_on):
    i1, i2, i3 = cue.Irreps("O3", "8x0e+8x1o"), cue.Irreps("O3", "0e+1o"), cue.Irreps("O3", "16x0e+16x1o")
    e = descriptors.fully_connected_tensor_product(i1, i2, i3)
    t = flattened_tables(e.polynomial)
    assert not jit._has_spec(t, 0)
    assert jit.ensure_specialised(t, 0, None, origin=e.polynomial)
    assert jit._has_spec(t, 0) and jit._has_spec(t.backward((True, True, True)), 0)


def run_case(device, ir1, ir2, ir3, N, Z, dtype, seed, indexed, sort_receivers=True):
    from cuequivariance_amd import cuet
    from oracle.naive import naive_segmented_polynomial, spec_from_polynomial

    i1, i2, i3 = (cue.Irreps("O3", s) for s in (ir1, ir2, ir3))
    m = cuet.FullyConnectedTensorProduct(i1, i2, i3, layout=cue.ir_mul, shared_weights=False, internal_weights=False,
                                         device=device, dtype=dtype)
    spec = spec_from_polynomial(descriptors.fully_connected_tensor_product(i1, i2, i3).polynomial)
    g = torch.Generator().manual_seed(seed)
    x1 = torch.randn(N if indexed else Z, i1.dim, dtype=torch.float64, generator=g).to(dtype)
    x2 = torch.randn(Z, i2.dim, dtype=torch.float64, generator=g).to(dtype)
    w = torch.randn(Z, m.weight_numel, dtype=torch.float64, generator=g).to(dtype)
    snd = torch.randint(0, max(N, 1), (Z,), generator=g, dtype=torch.int32)
    rcv = torch.randint(0, max(N, 1), (Z,), generator=g, dtype=torch.int32)
    if sort_receivers:
        rcv = torch.sort(rcv)[0]
    cot = torch.randn(N if indexed else Z, i3.dim, dtype=torch.float64, generator=g).to(dtype)
    a = [t.clone().requires_grad_(True) for t in (w, x1, x2)]
    ref = naive_segmented_polynomial(spec, a, {1: snd}, {0: N}, {0: rcv})[0] if indexed else naive_segmented_polynomial(spec, a)[0]
    ref_grads = torch.autograd.grad((ref * cot).sum(), a)
    b = [t.to(device).requires_grad_(True) for t in (w, x1, x2)]
    if indexed:
        out = m(b[1], b[2], b[0], indices_1=snd.to(device), indices_out=rcv.to(device), size_out=N)
    else:
        out = m(b[1], b[2], b[0])
    grads = torch.autograd.grad(out, b, cot.to(device))
    tol = 1e-12 if dtype == torch.float64 else 1e-5

    def close(got, want, what):
        got, want = got.detach().cpu().double(), want.double()
        err = (got - want).abs().max().item()
        assert err <= tol * max(want.abs().max().item(), 1e-30), f"{what}: {err:.3e}"

    close(out, ref, "out")
    for name, p, q in zip(("dw", "dx1", "dx2"), ref_grads, grads):
        close(q, p, name)
    return m


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("deterministic", ["0", "1"])
def test_row_weights_gather_scatter(device, dtype, deterministic, jit_on, monkeypatch):
    """64x0e+64x1o (x) 0e+1o+2e -> 64x0e+64x1o, 60 nodes / 700 edges, x1 gathered by sender, output summed by receiver."""
    monkeypatch.setenv("CUEQ_DETERMINISTIC", deterministic)
    m = run_case(device, "64x0e+64x1o", "0e+1o+2e", "64x0e+64x1o", 60, 700, dtype, seed=21, indexed=True)
    plan = m.f_per_sample.f.m._plan(dtype)
    assert plan.specialised(device) and plan.backward_plan((True, True, True)).specialised(device)
    assert jit._family(plan.tables, plan.polynomial, plan.origin) == "fc_rows"


@pytest.mark.gpu
def test_row_weights_plain_batch_and_unsorted_receivers(device, jit_on):
    run_case(device, "64x0e+64x1o", "0e+1o+2e", "64x0e+64x1o", 0, 300, torch.float32, seed=22, indexed=False)
    run_case(device, "64x0e+64x1o", "0e+1o+2e", "64x0e+64x1o", 500, 64, torch.float64, seed=23, indexed=True, sort_receivers=False)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_row_weights_multiplicities_below_the_wavefront(device, dtype, jit_on):
    """24 input and 40 output channels (lanes beyond them idle), outputs up to l = 2."""
    m = run_case(device, "24x0e+24x1o+24x2e", "0e+1o", "40x0e+40x1o+40x2e", 37, 333, dtype, seed=24, indexed=True)
    assert m.f_per_sample.f.m._plan(dtype).specialised(device)


@pytest.mark.gpu
def test_row_weights_without_batch_rows(device):
    """No edges at all: the output rows are zeros, the gradients have their shapes (the build's unit, no compilation)."""
    from cuequivariance_amd import cuet

    i1, i2 = cue.Irreps("O3", "64x0e+64x1o"), cue.Irreps("O3", "0e+1o+2e")
    m = cuet.FullyConnectedTensorProduct(i1, i2, i1, layout=cue.ir_mul, shared_weights=False, internal_weights=False,
                                         device=device, dtype=torch.float32)
    x1 = torch.randn(5, i1.dim, device=device, requires_grad=True)
    x2 = torch.randn(0, i2.dim, device=device, requires_grad=True)
    w = torch.randn(0, m.weight_numel, device=device, requires_grad=True)
    idx = torch.zeros(0, dtype=torch.int32, device=device)
    out = m(x1, x2, w, indices_1=idx, indices_out=idx, size_out=5)
    assert out.shape == (5, i1.dim) and float(out.detach().abs().sum()) == 0.0
    g1, g2, gw = torch.autograd.grad(out, [x1, x2, w], torch.ones_like(out))
    assert g1.shape == x1.shape and float(g1.abs().sum()) == 0.0 and g2.shape == x2.shape and gw.shape == w.shape
    assert m.f_per_sample.f.m._plan(torch.float32).specialised(device)
