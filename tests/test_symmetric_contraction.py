"""Symmetric contraction: reduced symmetric basis, descriptor, MACE parametrisation, module.

CPU tests pin the restated basis algorithm by what the reference's own tests and docs hold:
``cuequivariance/tests/group_theory/reduced_tensor_product_test.py:22-41`` (elasticity tensor, symmetric basis),
``cuequivariance/tests/group_theory/equivariant_polynomial_test.py:139-151`` (path counts 437 -> 105),
``cuequivariance/group_theory/descriptors/symmetric_contractions.py:110-120`` (doc example: 32+80+176 weights,
4/37/437 paths), ``cuequivariance/tests/group_theory/experimental/mace_test.py`` and
``experimental/mace/symmetric_contractions.py:37-40`` (projection shapes), and the golden vector of the ORIGINAL
MACE implementation that ``cuequivariance_torch/tests/operations/symmetric_contraction_test.py:77-124`` holds.
GPU tests compare the module with the CPU oracle (fp64 1e-12, fp32 1e-5 of max|ref|) and with that golden vector.
"""

import base64
import itertools
import json
from pathlib import Path

import numpy as np
import pytest
import torch

from cuequivariance_amd import cue
from oracle.naive import naive_segmented_polynomial, spec_from_polynomial

GOLDEN = Path(__file__).parent / "golden" / "mace_symmetric_contraction.json"


def test_elasticity_tensor_has_21_components():
    C = cue.reduced_tensor_product_basis("ijkl=klij=jikl", i=cue.Irreps("O3", "1o"))
    assert C.shape == (3, 3, 3, 3, 21)


def test_symmetric_basis_is_symmetric_and_independent():
    C = cue.reduced_symmetric_tensor_product_basis(cue.Irreps("SU2", "1/2 + 1"), 4).array
    assert C.shape == (5, 5, 5, 5, 70)
    for perm in itertools.permutations(range(4)):
        np.testing.assert_array_equal(C, np.transpose(C, perm + (4,)))
    assert np.linalg.matrix_rank(np.reshape(C, (5**4, 70))) == 70


def test_antisymmetric_basis_dimension():
    # Lambda^2 of a 3-vector is a pseudo-vector: one 1e
    C = cue.reduced_antisymmetric_tensor_product_basis(cue.Irreps("O3", "1o"), 2)
    assert C.irreps == cue.Irreps("O3", "1e") and C.shape == (3, 3, 3)
    np.testing.assert_allclose(C.array, -np.transpose(C.array, (1, 0, 2)))


def test_symmetric_square_of_vector_matches_closed_form():
    # Sym^2(1o) = 0e + 2e; the 0e part is delta_ij / sqrt(3) up to sign
    C = cue.reduced_symmetric_tensor_product_basis(cue.Irreps("O3", "1o"), 2)
    assert C.irreps == cue.Irreps("O3", "0e + 2e")
    np.testing.assert_allclose(np.abs(C.array[:, :, 0]), np.eye(3) / np.sqrt(3), atol=1e-12)
    flat = C.array.reshape(9, 6)
    np.testing.assert_allclose(flat.T @ flat, np.eye(6), atol=1e-12)


def test_descriptor_doc_example_counts():
    e = cue.descriptors.symmetric_contraction(
        16 * cue.Irreps("SO3", "0 + 1 + 2"), 16 * cue.Irreps("SO3", "0 + 1"), (1, 2, 3)
    )
    p = e.polynomial
    assert p.inputs[0].size == 288 and p.inputs[0].num_segments == 32 // 16 + 80 // 16 + 176 // 16
    assert [d.num_paths for _, d in p.operations] == [4, 37, 437]
    assert [tuple(o.buffers) for o, _ in p.operations] == [(0, 1, 2), (0, 1, 1, 2), (0, 1, 1, 1, 2)]
    assert p.all_same_segment_shape()


def test_descriptor_with_degree_zero_and_unsymmetrize():
    e = cue.descriptors.symmetric_contraction(
        16 * cue.Irreps("SO3", "0 + 1 + 2"), 16 * cue.Irreps("SO3", "0 + 1"), [0, 1, 2, 3]
    )
    assert e.polynomial.num_inputs == 2 and e.polynomial.num_outputs == 1
    assert e.polynomial.operations[3][1].num_paths == 437
    assert e.polynomial.unsymmetrize_for_identical_operands().operations[3][1].num_paths == 105


def test_descriptor_is_equivariant_and_symmetric():
    """O(3) equivariance of the numpy evaluation under a random rotation (Wigner matrices from the generators)."""
    from scipy.linalg import expm

    irreps_in, irreps_out = cue.Irreps("O3", "2x0e + 2x1o + 2x2e"), cue.Irreps("O3", "2x0e + 2x1o")
    e = cue.descriptors.symmetric_contraction(irreps_in, irreps_out, (1, 2, 3))
    rng = np.random.default_rng(0)
    angles = rng.normal(size=3)

    def rep(irreps):  # block-diagonal representation matrix in ir_mul layout
        blocks = []
        for mul, ir in irreps:
            X = ir.continuous_generators()
            D = expm(np.einsum("a,aij->ij", angles, X))
            blocks.append(np.kron(D, np.eye(mul)))
        n = sum(b.shape[0] for b in blocks)
        out, o = np.zeros((n, n)), 0
        for b in blocks:
            out[o: o + b.shape[0], o: o + b.shape[0]] = b
            o += b.shape[0]
        return out

    w = rng.normal(size=e.polynomial.inputs[0].size)
    x = rng.normal(size=irreps_in.dim)
    [y] = e.polynomial(w, x)
    [y_rot] = e.polynomial(w, rep(irreps_in) @ x)
    np.testing.assert_allclose(y_rot, rep(irreps_out) @ y, atol=1e-10)


def test_mace_projection_shapes():
    e, p = cue.mace.symmetric_contraction(4 * cue.Irreps("SO3", "0+1+2"), 4 * cue.Irreps("SO3", "0+1"), [1, 2, 3])
    assert p.shape == (62, 18)
    e, p = cue.mace.symmetric_contraction(
        cue.Irreps("O3", "32x0e + 32x1o"), cue.Irreps("O3", "32x0e + 32x1o"), degrees=[1, 2, 3]
    )
    assert p.shape[1] == e.inputs[0].dim // 32


def _golden():
    g = json.loads(GOLDEN.read_text())

    def arr(d):
        a = np.frombuffer(base64.b64decode(d["float32_base64"]), dtype=np.float32).reshape(d["shape"])
        return torch.from_numpy(a.copy())

    return g, arr(g["x"]), arr(g["weight"]), arr(g["expected_output"]), torch.tensor(g["indices"], dtype=torch.int32)


def _golden_module(g, device=None):
    from cuequivariance_amd import cuet

    return cuet.SymmetricContraction(
        g["mul"] * cue.Irreps(cue.O3_e3nn, g["irreps_in"]), g["mul"] * cue.Irreps(cue.O3_e3nn, g["irreps_out"]),
        contraction_degree=g["contraction_degree"], num_elements=g["num_elements"], layout_in=cue.ir_mul,
        layout_out=cue.mul_ir, original_mace=True, device=device, dtype=torch.float32, math_dtype=torch.float64,
    )


def test_oracle_reproduces_original_mace_output():
    g, x, w, expected, idx = _golden()
    m = _golden_module(g)
    assert tuple(m.weight.shape) == tuple(w.shape)
    weight = torch.einsum("zau,ab->zbu", w.double(), m.projection.double()).flatten(1)
    out = naive_segmented_polynomial(spec_from_polynomial(m.etp.polynomial), [weight, x.double()], {0: idx})[0]
    # the golden vector is in the mul_ir layout; the oracle works in ir_mul: per-segment (ir, mul) -> (mul, ir) by views
    parts, off = [], 0
    for mul, ir in m.irreps_out:
        parts.append(out[:, off: off + mul * ir.dim].reshape(-1, ir.dim, mul).transpose(1, 2).reshape(-1, mul * ir.dim))
        off += mul * ir.dim
    torch.testing.assert_close(torch.cat(parts, dim=1).float(), expected, atol=g["atol"], rtol=g["rtol"])


@pytest.mark.gpu
def test_module_reproduces_original_mace_output(device):
    g, x, w, expected, idx = _golden()
    m = _golden_module(g, device)
    m.weight.data = w.to(device)
    out = m(x.to(device), idx.to(device))
    torch.testing.assert_close(out.cpu(), expected, atol=g["atol"], rtol=g["rtol"])


@pytest.mark.gpu
@pytest.mark.parametrize(
    "irreps_in,irreps_out,degree,nel,Z,dtype,tol,original_mace",
    [
        ("32x0e+32x1o", "32x0e", 3, 5, 100, torch.float64, 1e-12, False),
        ("32x0e+32x1o+32x2e", "32x0e+32x1o", 3, 4, 257, torch.float32, 1e-5, False),
        ("16x0e+16x1o+16x2e+16x3o", "16x0e+16x1o", 3, 10, 64, torch.float64, 1e-12, False),
        ("8x0e+8x1o+8x2e", "8x0e+8x1o", 2, 3, 33, torch.float64, 1e-12, True),
        ("128x0e+128x1o+128x2e+128x3o", "128x0e+128x1o", 3, 10, 40, torch.float32, 1e-5, False),
    ],
)
def test_module_matches_oracle(device, irreps_in, irreps_out, degree, nel, Z, dtype, tol, original_mace):
    from cuequivariance_amd import cuet

    m = cuet.SymmetricContraction(
        cue.Irreps("O3", irreps_in), cue.Irreps("O3", irreps_out), degree, nel, layout=cue.ir_mul,
        dtype=torch.float64, original_mace=original_mace,
    )
    gen = torch.Generator().manual_seed(1)
    x = torch.randn(Z, m.irreps_in.dim, dtype=torch.float64, generator=gen).to(dtype).double()
    idx = torch.randint(0, nel, (Z,), generator=gen, dtype=torch.int32)
    w = m.weight.detach().clone()
    if original_mace:
        w = torch.einsum("zau,ab->zbu", w, m.projection)
    w = w.flatten(1).to(dtype).double()
    a = [w.clone().requires_grad_(True), x.clone().requires_grad_(True)]
    ref = naive_segmented_polynomial(spec_from_polynomial(m.etp.polynomial), a, {0: idx})[0]
    cot = torch.randn(ref.shape, dtype=torch.float64, generator=gen).to(dtype).double()
    ref_grads = torch.autograd.grad(ref, a, cot)
    b = [t.to(dtype).to(device).requires_grad_(True) for t in (w, x)]
    out = m.f(b, input_indices={0: idx.to(device)})[0]
    grads = torch.autograd.grad(out, b, cot.to(dtype).to(device))
    for name, got, want in [("out", out, ref), ("dw", grads[0], ref_grads[0]), ("dx", grads[1], ref_grads[1])]:
        err = (got.double().cpu() - want).abs().max().item()
        assert err <= tol * want.abs().max().item(), (name, err, want.abs().max().item())


@pytest.mark.gpu
def test_module_forward_signature_and_layouts(device):
    from cuequivariance_amd import cuet

    irreps_in, irreps_out = cue.Irreps("O3", "8x0e+8x1o"), cue.Irreps("O3", "8x0e+8x1o")
    a = cuet.SymmetricContraction(irreps_in, irreps_out, 2, 3, layout=cue.ir_mul, device=device, dtype=torch.float32)
    b = cuet.SymmetricContraction(irreps_in, irreps_out, 2, 3, layout=cue.mul_ir, device=device, dtype=torch.float32)
    b.weight.data = a.weight.data.clone()
    x = torch.randn(20, irreps_in.dim, device=device)
    idx = torch.randint(0, 3, (20,), device=device)  # int64 indices
    ya = a(x, idx)
    to_mul_ir = cuet.TransposeIrrepsLayout(irreps_in, source=cue.ir_mul, target=cue.mul_ir, device=device)
    yb = b(to_mul_ir(x), idx)
    torch.testing.assert_close(to_mul_ir(ya), yb, atol=1e-5, rtol=1e-5)
    with pytest.raises(ValueError):
        cuet.SymmetricContraction(cue.Irreps("O3", "8x0e+4x1o"), irreps_out, 2, 3, layout=cue.ir_mul)


@pytest.mark.gpu
def test_generated_kernels_full_size(device, monkeypatch):
    """cfg3 shape (50 000 nodes, 128 channels, l <= 3 -> 0e+1o, 10 element types): the descriptor-specialised kernels are
    the ones running, repeat bit-identically (no atomics in the weight gradient), and agree with the table-driven
    kernels on a slice; element types that never occur get a zero gradient; int64 and pre-sorted indices work."""
    from cuequivariance_amd import cuet

    m = cuet.SymmetricContraction(
        cue.Irreps("O3", "128x0e+128x1o+128x2e+128x3o"), cue.Irreps("O3", "128x0e+128x1o"), 3, 10, layout=cue.ir_mul,
        dtype=torch.float32, device=device,
    )
    plan = m.f.m._plan(torch.float32)
    assert plan.specialised(device) and plan.backward_plan((True, True)).specialised(device)
    assert plan.backward_plan((False, True)).specialised(device) and plan.backward_plan((True, False)).specialised(device)
    Z = 50_000
    gen = torch.Generator(device=device).manual_seed(0)
    x = torch.randn(Z, 2048, device=device, generator=gen, requires_grad=True)
    idx = torch.randint(0, 9, (Z,), device=device, generator=gen, dtype=torch.int32)  # type 9 never occurs
    cot = torch.randn(Z, 512, device=device, generator=gen)

    def step(xx, ii, cc):
        out = m(xx, ii)
        return [out] + list(torch.autograd.grad(out, [m.weight, xx], cc))

    a, b = step(x, idx, cot), step(x, idx, cot)
    for u, v in zip(a, b):
        assert torch.equal(u, v)
    assert torch.count_nonzero(a[1][9]) == 0 and torch.count_nonzero(a[1][3]) > 0
    # int64 indices; sorted indices (identity permutation in the grouping)
    c = step(x, idx.long(), cot)
    assert torch.equal(a[0], c[0]) and torch.equal(a[2], c[2])
    order = torch.sort(idx.long(), stable=True)[1]
    d = step(x[order].detach().requires_grad_(True), idx[order].contiguous(), cot[order].contiguous())
    assert torch.equal(d[0], a[0][order]) and torch.equal(d[2], a[2][order])
    assert (d[1] - a[1]).abs().max().item() <= 1e-5 * a[1].abs().max().item()
    # slice against the generic kernels
    Zs = 2000
    xs = x[:Zs].detach().requires_grad_(True)
    got = step(xs, idx[:Zs].contiguous(), cot[:Zs].contiguous())
    monkeypatch.setenv("CUEQ_FORCE_GENERIC", "1")
    want = step(xs, idx[:Zs].contiguous(), cot[:Zs].contiguous())
    for name, u, v in zip(("out", "dw", "dx"), got, want):
        assert (u - v).abs().max().item() <= 5e-5 * v.abs().max().item(), name
    # only the input gradient (frozen weights) and only the weight gradient
    monkeypatch.delenv("CUEQ_FORCE_GENERIC")
    out = m(xs, idx[:Zs].contiguous())
    (gx,) = torch.autograd.grad(out, [xs], cot[:Zs].contiguous(), retain_graph=True)
    (gw,) = torch.autograd.grad(out, [m.weight], cot[:Zs].contiguous())
    assert torch.equal(gx, got[2]) and torch.equal(gw, got[1])
