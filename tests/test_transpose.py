"""Segmented (u, v) -> (v, u) transposition on the GPU (``cueq_segmented_transpose``), the layout glue between
``mul_ir`` and ``ir_mul``.  Cases of the reference's own test
(``cuequivariance_torch/tests/primitives/transpose_test.py:31-67``: the 2x3 + 2x2 example and the empty tensor) plus
bit-exact agreement with the view-based definition, the backward, long rows and leading dimensions."""

import numpy as np
import pytest
import torch


def by_views(x, segments):
    outs, off = [], 0
    for u, v in segments:
        seg = x[..., off: off + u * v]
        outs.append(seg.reshape(x.shape[:-1] + (u, v)).transpose(-2, -1).reshape(x.shape[:-1] + (u * v,)))
        off += u * v
    return torch.cat(outs, dim=-1)


def test_permutation_table_is_the_documented_example():
    from cuequivariance_amd.cuet.transpose import _permutation

    # 1 2 3 / 4 5 6 -> 1 4 / 2 5 / 3 6 ; 10 11 / 12 13 -> 10 12 / 11 13   (reference transpose_test.py:33-52)
    x = np.array([1.0, 2, 3, 4, 5, 6, 10, 11, 12, 13])
    assert x[_permutation([(2, 3), (2, 2)])].tolist() == [1, 4, 2, 5, 3, 6, 10, 12, 11, 13]
    p = _permutation([(4, 3), (1, 5), (2, 2)])
    assert sorted(p.tolist()) == list(range(21))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16, torch.bfloat16])
def test_reference_example_and_empty(device, dtype):
    from cuequivariance_amd import cuet

    m = cuet.TransposeSegments([(2, 3), (2, 2)], device)
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 10, 11, 12, 13]], dtype=dtype, device=device)
    want = torch.tensor([[1.0, 4.0, 2.0, 5.0, 3.0, 6.0, 10, 12, 11, 13]], dtype=dtype, device=device)
    assert torch.equal(m(x), want)
    empty = torch.zeros((0, 10), dtype=dtype, device=device)
    assert m(empty).shape == (0, 10)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16])
@pytest.mark.parametrize("segments,lead", [
    ([(128, 1), (128, 3), (128, 5), (128, 7)], (1000,)),    # mul_ir -> ir_mul of 128x0e+128x1o+128x2e+128x3o
    ([(1, 128), (3, 128), (5, 128), (7, 128)], (3, 7, 11)),  # back, several leading dimensions
    ([(512, 7), (512, 7), (512, 7), (512, 7)], (40,)),       # 14336 elements: fp32 / fp64 rows exceed the LDS path
    ([(5, 4), (2, 6), (1, 9), (3, 3)], (257,)),
])
def test_bit_exact_against_views_and_backward(device, dtype, segments, lead):
    from cuequivariance_amd import cuet

    total = sum(u * v for u, v in segments)
    g = torch.Generator().manual_seed(total)
    x = torch.randn(*lead, total, generator=g).to(dtype).to(device).requires_grad_(True)
    m = cuet.TransposeSegments(segments, device)
    y = m(x)
    assert torch.equal(y, by_views(x.detach(), segments))
    cot = torch.randn(*lead, total, generator=g).to(dtype).to(device)
    (gx,) = torch.autograd.grad(y, [x], cot)
    assert torch.equal(gx, by_views(cot, [(v, u) for u, v in segments]))
    # the two layouts are inverse to each other
    back = cuet.TransposeSegments([(v, u) for u, v in segments], device)
    assert torch.equal(back(y.detach()), x.detach())
    # a non-contiguous view as input
    wide = torch.randn(*lead, 2 * total, generator=g).to(dtype).to(device)
    assert torch.equal(m(wide[..., ::2]), by_views(wide[..., ::2], segments))


@pytest.mark.gpu
def test_irreps_layout_module_and_errors(device):
    from cuequivariance_amd import cue, cuet

    irreps = cue.Irreps("O3", "32x0e+16x1o+8x2e")
    x = torch.randn(50, irreps.dim, device=device)
    to_ir_mul = cuet.TransposeIrrepsLayout(irreps, source=cue.mul_ir, target=cue.ir_mul, device=device)
    to_mul_ir = cuet.TransposeIrrepsLayout(irreps, source=cue.ir_mul, target=cue.mul_ir, device=device)
    assert torch.equal(to_ir_mul(x), by_views(x, [(mul, ir.dim) for mul, ir in irreps]))
    assert torch.equal(to_mul_ir(to_ir_mul(x)), x)
    same = cuet.TransposeIrrepsLayout(irreps, source=cue.ir_mul, target=cue.ir_mul, device=device)
    assert same(x) is x
    with pytest.raises(ValueError):
        to_ir_mul(x[:, :-1])
    with pytest.raises(ValueError):
        to_ir_mul(x.cpu())
    with pytest.raises(ValueError):
        cuet.TransposeSegments([(2, 3)], device, use_fallback=True)
