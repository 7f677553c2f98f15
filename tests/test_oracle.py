"""Pins the CPU oracle (``oracle/naive.py``) against what the mathematics fixes.

* brute-force loops over every index on tiny descriptors (a dropped path, a wrong segment offset
  or a transposed operand changes the result);
* textbook reductions: matrix product (the reference's ``evaluate_test.py:20-104``), the channel-wise
  product written directly from Clebsch-Gordan tensors;
* gather / scatter identity ``f(x[idx]) scattered == f(x, idx)`` including gradients
  (``cuequivariance_torch/tests/operations/channel_wise_test.py:231-305``);
* batch rules of the executor (one-row inputs broadcast, a one-row output sums over the batch,
  ``segmented_polynomial_naive.py:387-433``);
* casting rule for low-precision inputs (``:107-127``): operands are cast to ``math_dtype``, each
  path's result is cast back to the dtype of the first input before the paths are summed.
"""

import itertools

import numpy as np
import pytest
import torch

from cuequivariance_amd import cue
from oracle.naive import naive_segmented_polynomial, numpy_last_operand, spec_from_polynomial


def small_u1d_polynomial(u=3):
    d = cue.SegmentedTensorProduct.from_subscripts("u,u,,u")
    d.add_segments(0, [(u,)] * 2)
    d.add_segments(1, [(u,)] * 3)
    d.add_segments(2, [()] * 2)
    d.add_segments(3, [(u,)] * 2)
    paths = [(0, 2, 1, 0, 1.5), (1, 0, 0, 0, -2.0), (1, 1, 1, 1, 0.25), (0, 0, 0, 1, 3.0)]
    for a, b, c, o, coef in paths:
        d.add_path(a, b, c, o, c=coef)
    return cue.SegmentedPolynomial.eval_last_operand(d), paths


def test_brute_force_uniform1d():
    u = 3
    poly, paths = small_u1d_polynomial(u)
    rng = np.random.default_rng(0)
    Z = 5
    a, b, s = rng.normal(size=(Z, 2 * u)), rng.normal(size=(Z, 3 * u)), rng.normal(size=(Z, 2))
    expect = np.zeros((Z, 2 * u))
    for z in range(Z):
        for (ia, ib, is_, io, coef) in paths:
            for c in range(u):
                expect[z, io * u + c] += coef * a[z, ia * u + c] * b[z, ib * u + c] * s[z, is_]
    got = naive_segmented_polynomial(spec_from_polynomial(poly), [torch.tensor(a), torch.tensor(b), torch.tensor(s)])[0]
    np.testing.assert_allclose(got.numpy(), expect, rtol=1e-13, atol=1e-13)
    np.testing.assert_allclose(poly(a, b, s)[0], expect, rtol=1e-13, atol=1e-13)


def test_brute_force_with_coefficient_modes():
    rng = np.random.default_rng(1)
    d = cue.SegmentedTensorProduct.from_subscripts("uv,iu,jv,kuv+ijk")
    c0, c1 = rng.normal(size=(2, 3, 2)), rng.normal(size=(1, 3, 3))
    d.add_segment(1, (2, 2))
    d.add_segment(1, (1, 2))
    d.add_segment(2, (3, 1))
    d.add_path(None, 0, 0, None, c=c0, dims={"u": 2, "v": 1})
    d.add_path(None, 1, 0, None, c=c1, dims={"u": 2, "v": 1})
    poly = cue.SegmentedPolynomial.eval_last_operand(d)
    Z = 4
    w, x1, x2 = rng.normal(size=(Z, 4)), rng.normal(size=(Z, 6)), rng.normal(size=(Z, 3))
    expect = np.zeros((Z, d.operands[3].size))
    for z in range(Z):
        # path 0: w seg 0 (u=2,v=1) at 0..2, x1 seg 0 (i=2,u=2) at 0..4, out seg 0 (k=2,u=2,v=1) at 0..4
        for i, j, k, uu in itertools.product(range(2), range(3), range(2), range(2)):
            expect[z, k * 2 + uu] += c0[i, j, k] * w[z, uu] * x1[z, i * 2 + uu] * x2[z, j]
        # path 1: w seg 1 at 2..4, x1 seg 1 (i=1,u=2) at 4..6, out seg 1 (k=3,u=2) at 4..10
        for j, k, uu in itertools.product(range(3), range(3), range(2)):
            expect[z, 4 + k * 2 + uu] += c1[0, j, k] * w[z, 2 + uu] * x1[z, 4 + uu] * x2[z, j]
    spec = spec_from_polynomial(poly)
    got = naive_segmented_polynomial(spec, [torch.tensor(w), torch.tensor(x1), torch.tensor(x2)])[0].numpy()
    np.testing.assert_allclose(got, expect, rtol=1e-13, atol=1e-13)
    # the numpy twin and the flattened form agree too
    np.testing.assert_allclose(numpy_last_operand(spec["operations"][0], w, x1, x2), expect, rtol=1e-13, atol=1e-13)
    flat = spec_from_polynomial(poly.flatten_coefficient_modes().squeeze_modes())
    got = naive_segmented_polynomial(flat, [torch.tensor(w), torch.tensor(x1), torch.tensor(x2)])[0].numpy()
    np.testing.assert_allclose(got, expect, rtol=1e-13, atol=1e-13)


def test_matmul_identity():
    d = cue.SegmentedTensorProduct.from_subscripts("uv,vw,uw")
    d.add_path(None, None, None, c=1.0, dims={"u": 2, "v": 3, "w": 4})
    spec = spec_from_polynomial(cue.SegmentedPolynomial.eval_last_operand(d))
    x0, x1 = torch.randn(10, 6, dtype=torch.float64), torch.randn(10, 12, dtype=torch.float64)
    ref = (x0.reshape(10, 2, 3) @ x1.reshape(10, 3, 4)).reshape(10, -1)
    torch.testing.assert_close(naive_segmented_polynomial(spec, [x0, x1])[0], ref, rtol=1e-13, atol=1e-13)


def channelwise_closed_form(irreps1, irreps2, filt, w, x1, x2):
    """out block (i1, i2, ir3) = w[:, b, u] * sum_ij C[i,j,k] x1[:, i, u] x2[:, j]  in ir_mul layout, blocks sorted by ir3."""
    blocks = []
    o1 = 0
    for m1, ir1 in irreps1:
        o2 = 0
        for m2, ir2 in irreps2:
            assert m2 == 1
            for ir3 in ir1 * ir2:
                if ir3 in filt:
                    for cg in cue.clebsch_gordan(ir1, ir2, ir3):
                        a = x1[:, o1: o1 + ir1.dim * m1].reshape(-1, ir1.dim, m1)
                        b = x2[:, o2: o2 + ir2.dim]
                        blocks.append((ir3, len(blocks), np.einsum("ijk,ziu,zj->zku", cg, a, b), m1))
            o2 += ir2.dim
        o1 += ir1.dim * m1
    order = sorted(range(len(blocks)), key=lambda n: (blocks[n][0]._key(), n))
    outs, ow = [], 0
    for new, n in enumerate(order):
        ir3, _, t, m1 = blocks[n]
        outs.append((t * w[:, None, ow: ow + m1]).reshape(t.shape[0], -1))
        ow += m1
    return np.concatenate(outs, axis=1)


def test_channelwise_closed_form():
    irreps1, irreps2 = cue.Irreps("O3", "4x0e+4x1o+4x2e"), cue.Irreps("O3", "0e+1o+2e")
    filt = [cue.O3(0, 1), cue.O3(1, -1), cue.O3(2, 1)]
    e = cue.descriptors.channelwise_tensor_product(irreps1, irreps2, filt)
    rng = np.random.default_rng(5)
    Z = 7
    w, x1, x2 = (rng.normal(size=(Z, op.size)) for op in e.polynomial.inputs)
    ref = channelwise_closed_form(irreps1, irreps2, filt, w, x1, x2)
    for poly in [e.polynomial, e.polynomial.flatten_coefficient_modes().squeeze_modes()]:
        got = naive_segmented_polynomial(spec_from_polynomial(poly), [torch.tensor(w), torch.tensor(x1), torch.tensor(x2)])
        np.testing.assert_allclose(got[0].numpy(), ref, rtol=1e-12, atol=1e-12)


def test_gather_scatter_identity_with_gradients():
    e = cue.descriptors.channelwise_tensor_product(cue.Irreps("O3", "3x0e+3x1o"), cue.Irreps("O3", "0e+1o"), "0e+1o")
    spec = spec_from_polynomial(e.polynomial)
    g = torch.Generator().manual_seed(0)
    N, Z = 6, 20
    w = torch.randn(Z, e.inputs[0].dim, dtype=torch.float64, generator=g, requires_grad=True)
    x1 = torch.randn(N, e.inputs[1].dim, dtype=torch.float64, generator=g, requires_grad=True)
    x2 = torch.randn(Z, e.inputs[2].dim, dtype=torch.float64, generator=g, requires_grad=True)
    snd = torch.randint(0, N, (Z,), generator=g, dtype=torch.int32)
    rcv = torch.randint(0, N, (Z,), generator=g)
    cot = torch.randn(N, e.outputs[0].dim, dtype=torch.float64, generator=g)
    out = naive_segmented_polynomial(spec, [w, x1, x2], {1: snd}, {0: N}, {0: rcv})[0]
    grads = torch.autograd.grad((out * cot).sum(), [w, x1, x2])
    dense = naive_segmented_polynomial(spec, [w, x1[snd.long()], x2])[0]
    out2 = torch.zeros(N, dense.shape[1], dtype=torch.float64).index_add(0, rcv, dense)
    grads2 = torch.autograd.grad((out2 * cot).sum(), [w, x1, x2])
    torch.testing.assert_close(out, out2, rtol=1e-13, atol=1e-13)
    for a, b in zip(grads, grads2):
        torch.testing.assert_close(a, b, rtol=1e-12, atol=1e-12)


def test_batch_rules():
    poly, _ = small_u1d_polynomial(2)
    spec = spec_from_polynomial(poly)
    Z = 6
    a, b, s = torch.randn(Z, 4, dtype=torch.float64), torch.randn(1, 6, dtype=torch.float64), torch.randn(Z, 2, dtype=torch.float64)
    full = naive_segmented_polynomial(spec, [a, b.expand(Z, 6), s])[0]
    torch.testing.assert_close(naive_segmented_polynomial(spec, [a, b, s])[0], full)  # one-row input broadcasts
    summed = naive_segmented_polynomial(spec, [a, b, s], output_shapes={0: 1})[0]
    torch.testing.assert_close(summed, full.sum(0, keepdim=True))  # one-row output sums the batch
    allshared = naive_segmented_polynomial(spec, [a[:1], b, s[:1]], output_shapes={0: 3})[0]
    torch.testing.assert_close(allshared, full[:1].expand(3, 4))  # one-row result broadcast to the requested rows
    with pytest.raises(ValueError):
        naive_segmented_polynomial(spec, [a, b[:, :5], s])


def test_low_precision_casting_rule():
    poly, paths = small_u1d_polynomial(2)
    spec = spec_from_polynomial(poly)
    g = torch.Generator().manual_seed(1)
    a, b, s = (torch.randn(4, n, generator=g).to(torch.bfloat16) for n in (4, 6, 2))
    got = naive_segmented_polynomial(spec, [a, b, s], math_dtype=torch.float32)[0]
    assert got.dtype == torch.bfloat16
    u = 2
    expect = torch.zeros(4, 4, dtype=torch.bfloat16)
    seen = set()
    for (ia, ib, is_, io, coef) in paths:
        term = (torch.tensor(coef, dtype=torch.float32) * a[:, ia * u:(ia + 1) * u].float() * b[:, ib * u:(ib + 1) * u].float()
                * s[:, is_:is_ + 1].float()).to(torch.bfloat16)
        if io in seen:
            expect[:, io * u:(io + 1) * u] = expect[:, io * u:(io + 1) * u] + term
        else:
            expect[:, io * u:(io + 1) * u] = term
            seen.add(io)
    torch.testing.assert_close(got.float(), expect.float(), rtol=1e-2, atol=1e-2)
