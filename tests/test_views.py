"""Operand views the kernels' fast paths do not take as they are - rows that start 4 bytes off a 16-byte boundary,
rows with a column stride, index tensors with a stride, empty batches: every module has to give what it gives on plain
contiguous copies (bit for bit where the same kernels run, to the dtype's tolerance where a slower path takes over)."""

import pytest
import torch

from cuequivariance_amd import cue

pytestmark = pytest.mark.gpu


def off_by_one(t):
    flat = torch.empty(t.numel() + 1, dtype=t.dtype, device=t.device)
    v = flat[1:].view(t.shape)
    v.copy_(t)
    return v


def column_strided(t):
    if t.dim() != 2:
        return t
    big = torch.empty(t.shape[0], 2 * t.shape[1] + 3, dtype=t.dtype, device=t.device)
    v = big[:, 3:3 + 2 * t.shape[1]:2]
    v.copy_(t)
    return v


def cases(device):
    from cuequivariance_amd import cuet

    g = torch.Generator(device=device).manual_seed(0)
    r = lambda *shape: torch.randn(*shape, device=device, generator=g)
    ir = cue.Irreps("O3", "64x0e+64x1o")
    lin = cuet.Linear(ir, ir, layout=cue.ir_mul, internal_weights=False, method="fused_tp")
    yield "Linear", (lambda x, w: lin(x, w)), [r(300, ir.dim), r(1, lin.weight_numel)]
    fc = cuet.FullyConnectedTensorProduct(cue.Irreps("O3", "8x0e+8x1o"), cue.Irreps("O3", "0e+1o"), cue.Irreps("O3", "8x0e+8x1o"),
                                          layout=cue.ir_mul, internal_weights=False)
    yield "FullyConnected", (lambda x1, x2, w: fc(x1, x2, w)), [r(70, 32), r(70, 4), r(1, fc.weight_numel)]
    i1, i2 = cue.Irreps("O3", "32x0e+32x1o+32x2e"), cue.Irreps("O3", "0e+1o+2e")
    cw = cuet.ChannelWiseTensorProduct(i1, i2, "0e+1o+2e", layout=cue.ir_mul, shared_weights=False)
    N, Z = 50, 600
    pairs = torch.stack([torch.randint(0, N, (Z,), device=device, generator=g),
                         torch.sort(torch.randint(0, N, (Z,), device=device, generator=g))[0]], 1)  # strided index columns
    yield ("ChannelWise indexed", (lambda x1, x2, w: cw(x1, x2, w, indices_1=pairs[:, 0], indices_out=pairs[:, 1], size_out=N)),
           [r(N, i1.dim), r(Z, i2.dim), r(Z, cw.weight_numel)])
    sc = cuet.SymmetricContraction(i1, cue.Irreps("O3", "32x0e+32x1o"), 3, 5, layout_in=cue.ir_mul, layout_out=cue.ir_mul,
                                   dtype=torch.float32, device=device)
    idx = torch.randint(0, 5, (200, 2), device=device, generator=g)
    yield "SymmetricContraction", (lambda x: sc(x, idx[:, 0])), [r(200, i1.dim) * 0.5]


@pytest.mark.parametrize("view", [off_by_one, column_strided])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_modules_take_unaligned_and_strided_views(device, dtype, view):
    for name, f, args in cases(device):
        if dtype == torch.bfloat16 and name in ("ChannelWise indexed", "SymmetricContraction"):
            continue  # (their bf16 I/O is covered elsewhere; the modules here were built for float32 math on float32 weights)
        args = [a.to(dtype) for a in args]
        a = [t.clone().requires_grad_(True) for t in args]
        out = f(*a)
        cot = torch.ones_like(out)
        want = (out,) + torch.autograd.grad(out, a, cot)
        b = [view(t).detach().requires_grad_(True) for t in args]
        out2 = f(*b)
        got = (out2,) + torch.autograd.grad(out2, b, view(cot))
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        for i, (u, v) in enumerate(zip(got, want)):
            assert u.shape == v.shape
            err = (u.float() - v.float()).abs().max().item() / max(v.float().abs().max().item(), 1e-30)
            assert err <= tol, (name, i, err)


def test_modules_take_empty_batches(device):
    for name, f, args in cases(device):
        if name == "ChannelWise indexed":
            continue  # (its batch is tied to the index tensors; empty indexed calls are covered in test_gpu_uniform1d.py)
        rows = args[0].shape[0]
        a = [(t[:0] if t.shape[0] == rows else t).clone().requires_grad_(True) for t in args]
        if name == "SymmetricContraction":
            continue  # (the element index is part of the closure; covered in test_symmetric_contraction.py)
        out = f(*a)
        assert out.shape[0] == 0
        grads = torch.autograd.grad(out, a, torch.ones_like(out), allow_unused=True)
        for t, gr in zip(a, grads):
            assert gr is None or (gr.shape == t.shape and (gr.numel() == 0 or gr.abs().max().item() == 0))
