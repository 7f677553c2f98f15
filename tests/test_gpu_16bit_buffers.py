"""Generated uniform-1d kernels with buffers of 16-bit elements (bfloat16, half) and float32 arithmetic.

The reference runs ``math_dtype=float32`` on tensors of any floating type
(``cuequivariance_torch/primitives/segmented_polynomial_uniform_1d.py:254-260``; its test matrix pairs float16 / bfloat16
tensors with float32 arithmetic, ``cuequivariance_torch/tests/primitives/segmented_polynomial_test.py:270-280``).  Here the
generated kernels exist per element type of the buffers; these tests check them against the float64 oracle evaluated on
the rounded inputs and make sure, through the kernel timers, that the generated kernels (not the table-driven ones) ran.

Tolerance (max-norm, relative to ``max|ref|``): 2e-2 for both 16-bit types: results are rounded once, to 8 (bfloat16) or
11 (half) bits, and sums of up to a few hundred such terms are formed in float32.
"""

import pytest
import torch

from cuequivariance_amd import _lib, cue
from oracle.naive import naive_segmented_polynomial, spec_from_polynomial

from test_gpu_uniform1d import assert_close, cw_module, run_cw_case

pytestmark = pytest.mark.gpu

TOL = 2e-2


def timed(fn):
    _lib.timing_begin()
    try:
        out = fn()
        torch.cuda.synchronize()
    finally:
        names = _lib.timing_end()
    return out, names


@pytest.mark.parametrize("deterministic", ["0", "1"])
def test_registered_channelwise_bfloat16(device, deterministic, monkeypatch):
    """The headline descriptor (128 channels, l <= 3) with gather and scatter, both policies for the gathered operand's
    gradient: the kernels linked into the library for bfloat16 buffers serve forward and backward."""
    monkeypatch.setenv("CUEQ_DETERMINISTIC", deterministic)
    m = cw_module("128x0e+128x1o+128x2e+128x3o", "0e+1o+2e+3o", "0e+1o+2e+3o")
    _, names = timed(lambda: run_cw_case(device, m, N=300, Z=4000, dtype=torch.bfloat16, seed=1, tol=TOL))
    assert "c128_l3_fwd_bf16" in names and "c128_l3_bwd_bf16" in names, names
    plan = m.f.m._plan(torch.float32)
    assert plan.math_dtype == torch.float32 and plan.serves(torch.bfloat16)
    assert plan.backward_plan((True, True, True)).serves(torch.bfloat16)


def test_registered_channelwise_bfloat16_batched_rows(device):
    """No gather, no scatter (one output row per batch row), 64 rows more than a multiple of the wavefront ranges."""
    m = cw_module("128x0e+128x1o+128x2e+128x3o", "0e+1o+2e+3o", "0e+1o+2e+3o")
    spec = spec_from_polynomial(m.f._polynomial_orig)
    g = torch.Generator().manual_seed(4)
    Z = 1000
    w, x1, x2 = (torch.randn(Z, n, dtype=torch.float64, generator=g).to(torch.bfloat16) for n in (m.weight_numel, m.irreps_in1.dim, m.irreps_in2.dim))
    cot = torch.randn(Z, m.irreps_out.dim, dtype=torch.float64, generator=g).to(torch.bfloat16)
    a = [t.double().requires_grad_(True) for t in (w, x1, x2)]
    ref = naive_segmented_polynomial(spec, a)[0]
    ref_grads = torch.autograd.grad(ref, a, cot.double())
    b = [t.to(device).requires_grad_(True) for t in (w, x1, x2)]

    def run():
        out = m(b[1], b[2], b[0])
        return out, torch.autograd.grad(out, b, cot.to(device))

    (out, grads), names = timed(run)
    assert "c128_l3_fwd_bf16" in names and "c128_l3_bwd_bf16" in names, names
    assert out.dtype == torch.bfloat16 and all(q.dtype == torch.bfloat16 for q in grads)
    assert_close(out, ref, TOL, "out")
    for name, p, q in zip(("dw", "dx1", "dx2"), ref_grads, grads):
        assert_close(q, p, TOL, name)


def test_registered_channelwise_mul_ir_bfloat16(device):
    from cuequivariance_amd import cuet

    m = cuet.ChannelWiseTensorProduct(cue.Irreps("O3", "128x0e+128x1o+128x2e+128x3o"), cue.Irreps("O3", "0e+1o+2e+3o"), "0e+1o+2e+3o",
                                      layout=cue.mul_ir, shared_weights=False)
    g = torch.Generator().manual_seed(6)
    N, Z = 200, 3000
    x1 = torch.randn(N, m.irreps_in1.dim, dtype=torch.float64, generator=g).to(torch.bfloat16)
    x2 = torch.randn(Z, m.irreps_in2.dim, dtype=torch.float64, generator=g).to(torch.bfloat16)
    w = torch.randn(Z, m.weight_numel, dtype=torch.float64, generator=g).to(torch.bfloat16)
    snd = torch.randint(0, N, (Z,), generator=g).to(torch.int32)
    rcv = torch.sort(torch.randint(0, N, (Z,), generator=g))[0].to(torch.int32)
    cot = torch.randn(N, m.irreps_out.dim, dtype=torch.float64, generator=g).to(torch.bfloat16)

    def run(mod, dtype):
        b = [t.to(device=device, dtype=dtype).requires_grad_(True) for t in (w, x1, x2)]
        out = mod(b[1], b[2], b[0], indices_1=snd.to(device), indices_out=rcv.to(device), size_out=N)
        return out, torch.autograd.grad(out, b, cot.to(device=device, dtype=dtype))

    # the float64 kernels of the same module on the same (rounded) mul_ir rows are the reference here: they are checked
    # against the oracle by the tests of the layouts
    (out, grads), names = timed(lambda: run(m, torch.bfloat16))
    assert "c128_l3_mulir_fwd_bf16" in names and "c128_l3_mulir_bwd_bf16" in names, names
    ref, ref_grads = run(m, torch.float64)
    assert_close(out, ref, TOL, "out")
    for name, p, q in zip(("dw", "dx1", "dx2"), ref_grads, grads):
        assert_close(q, p, TOL, name)


@pytest.mark.parametrize("layout", [cue.ir_mul, cue.mul_ir])
def test_registered_symmetric_contraction_bfloat16(device, layout):
    from cuequivariance_amd import cuet

    irreps_in, irreps_out = cue.Irreps("O3", "128x0e+128x1o+128x2e+128x3o"), cue.Irreps("O3", "128x0e+128x1o")
    m = cuet.SymmetricContraction(irreps_in, irreps_out, 3, 10, layout=layout, device=device, dtype=torch.float32)
    g = torch.Generator().manual_seed(8)
    Z = 900
    x = torch.randn(Z, irreps_in.dim, dtype=torch.float64, generator=g).to(torch.bfloat16)
    idx = torch.randint(0, 10, (Z,), generator=g).to(torch.int32)
    cot = torch.randn(Z, irreps_out.dim, dtype=torch.float64, generator=g).to(torch.bfloat16)
    assert m.projection is None
    wq = m.weight.detach().to(torch.bfloat16)  # the weights, rounded once: both runs see the same values

    def run(dtype):
        ww = wq.to(dtype).requires_grad_(True)
        xx = x.to(device=device, dtype=dtype).requires_grad_(True)
        out = _call(m, ww, xx, idx.to(device))
        gw, gx = torch.autograd.grad(out, [ww, xx], cot.to(device=device, dtype=dtype))
        return out, gw, gx

    (out, gw, gx), names = timed(lambda: run(torch.bfloat16))
    tag = "s128_l3_mulir" if layout == cue.mul_ir else "s128_l3"
    assert f"{tag}_fwd_bf16" in names and any(k.startswith(f"{tag}_bwd_") and k.endswith("_bf16") for k in names), names
    ref, rw, rx = run(torch.float64)
    assert out.dtype == torch.bfloat16
    assert_close(out, ref, TOL, "out")
    assert_close(gw, rw, TOL, "dw")
    assert_close(gx, rx, TOL, "dx")


def _call(m, w, x, idx):
    """The module's computation with the weights given from outside (its own parameter holds float32)."""
    import torch.func

    return torch.func.functional_call(m, {"weight": w}, (x, idx))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_compiled_at_first_use_for_16bit_buffers(device, dtype):
    """A descriptor the library has no 16-bit kernels for (32 channels, l <= 2) gets them at first use: the channel-wise unit
    (forward and fused backward) for exactly the element type of the call."""
    from cuequivariance_amd import jit

    was = jit.enabled()
    jit.enable(True)
    try:
        m = cw_module("32x0e+32x1o+32x2e", "0e+1o+2e", "0e+1o+2e")
        _, names = timed(lambda: run_cw_case(device, m, N=100, Z=1500, dtype=dtype, seed=3, tol=TOL))
        tag = "bf16" if dtype == torch.bfloat16 else "f16"
        assert any(k.endswith(f"_fwd_{tag}") for k in names) and any(k.endswith(f"_bwd_{tag}") for k in names), names
        plan = m.f.m._plan(torch.float32)
        assert plan.serves(dtype) and plan.backward_plan((True, True, True)).serves(dtype)
    finally:
        jit.enable(was)


def test_general_unit_for_16bit_buffers(device):
    """A plan outside the generated families (spherical harmonics of degree <= 3) with bfloat16 buffers: the general generator's
    unit for that element type."""
    from cuequivariance_amd import cuet, jit

    was = jit.enabled()
    jit.enable(True)
    try:
        sh = cuet.SphericalHarmonics([0, 1, 2, 3], normalize=False, device=device)
        v = torch.randn(700, 3, dtype=torch.float64, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16)
        out, names = timed(lambda: sh(v.to(device)))
        ref = sh(v.double().to(device))
        assert out.dtype == torch.bfloat16
        assert any(k.endswith("_bf16") for k in names), names
        assert_close(out, ref, TOL, "harmonics")
    finally:
        jit.enable(was)
