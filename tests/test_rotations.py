"""Rotations and the inversion of SO(3) / O(3) features (reference descriptors
``cuequivariance/group_theory/descriptors/rotations.py:23-252``, modules ``cuequivariance_torch/operations/rotation.py:29-310``).

The descriptors here are derived from the generators of the irreps, so they are pinned by what a rotation must do, not by a
copy of the reference's tables: on vectors (``1o``, components x, y, z) they are the textbook right-handed rotation matrices
about y and x in the order the reference documents (``R = R_y(alpha) R_x(beta) R_y(gamma)``; ``vector_to_euler_angles`` solves
``R_y(alpha) R_x(beta) e_y = v``); on higher degrees they commute with the spherical harmonics (``Y(R v) = D(R) Y(v)``), which
fixes every sign and axis convention; the y rotation has the ``1 + 4 l`` paths per irrep that the reference's construction gives;
the inversion is the parity and ``Y_l(-v) = (-1)^l Y_l(v)``.
"""

import numpy as np
import pytest
import torch

from cuequivariance_amd import cue
from cuequivariance_amd.cue import descriptors
from oracle.naive import naive_segmented_polynomial, spec_from_polynomial


def Ry(t):
    c, s = np.cos(t), np.sin(t)
    return np.array([[c, 0, s], [0, 1, 0], [-s, 0, c]])  # z towards x


def Rx(t):
    c, s = np.cos(t), np.sin(t)
    return np.array([[1, 0, 0], [0, c, -s], [0, s, c]])  # y towards z


def encode(t, L):
    m = np.arange(1, L + 1)
    return np.concatenate([np.cos(t * m[::-1]), [1.0], np.sin(t * m)])[None, :]


def change_layout(x, irreps, to_ir_mul: bool):
    """``mul_ir`` rows (channel outside, component inside) to ``ir_mul`` rows or back, irrep by irrep (differentiable)."""
    out, off = [], 0
    for mul, ir in irreps:
        block = x[:, off:off + mul * ir.dim]
        block = block.reshape(-1, mul, ir.dim) if to_ir_mul else block.reshape(-1, ir.dim, mul)
        out.append(block.transpose(1, 2).reshape(x.shape[0], -1))
        off += mul * ir.dim
    return torch.cat(out, 1)


def evaluate(e, *inputs):
    return naive_segmented_polynomial(spec_from_polynomial(e.polynomial), [torch.as_tensor(np.asarray(a, dtype=np.float64)) for a in inputs])[0].numpy()


def test_rotations_of_vectors_are_the_textbook_matrices():
    irreps = cue.Irreps("O3", "1x1o")
    g, b, a = 0.37, -1.21, 2.05
    v = np.random.default_rng(0).normal(size=(5, 3))
    assert np.allclose(evaluate(descriptors.y_rotation(irreps), encode(g, 1), v), v @ Ry(g).T, atol=1e-12)
    assert np.allclose(evaluate(descriptors.x_rotation(irreps), encode(b, 1), v), v @ Rx(b).T, atol=1e-12)
    assert np.allclose(evaluate(descriptors.xy_rotation(irreps), encode(g, 1), encode(b, 1), v), v @ (Rx(b) @ Ry(g)).T, atol=1e-12)
    assert np.allclose(evaluate(descriptors.yx_rotation(irreps), encode(b, 1), encode(g, 1), v), v @ (Ry(g) @ Rx(b)).T, atol=1e-12)
    assert np.allclose(evaluate(descriptors.yxy_rotation(irreps), encode(g, 1), encode(b, 1), encode(a, 1), v),
                       v @ (Ry(a) @ Rx(b) @ Ry(g)).T, atol=1e-12)
    axis = np.array([0.3, -0.5, 0.8])
    axis /= np.linalg.norm(axis)
    K = np.array([[0, -axis[2], axis[1]], [axis[2], 0, -axis[0]], [-axis[1], axis[0], 0]])
    R = np.eye(3) + np.sin(0.7) * K + (1 - np.cos(0.7)) * K @ K  # Rodrigues
    assert np.allclose(evaluate(descriptors.fixed_axis_angle_rotation(irreps, axis, 0.7), v), v @ R.T, atol=1e-12)


@pytest.mark.parametrize("group", ["SO3", "O3"])
def test_rotations_commute_with_the_spherical_harmonics(group):
    """``Y_l(R v) = D_l(R) Y_l(v)`` for l = 0..4 with multiplicity 2 (two different vectors side by side, ``ir_mul`` rows), for
    the single rotations, their compositions with a larger ``lmax`` than needed, and a rotation about a general axis."""
    ls = [0, 1, 2, 3, 4]
    vec_ir = cue.SO3(1) if group == "SO3" else cue.O3(1, -1)
    irreps = cue.Irreps(group, [(2, cue.SO3(l) if group == "SO3" else cue.O3(l, (-1) ** l)) for l in ls])
    rng = np.random.default_rng(1)
    v = rng.normal(size=(2, 3))

    def features(vectors):  # (irrep, component, multiplicity) rows
        Y = descriptors.spherical_harmonics_values(vec_ir, ls, vectors)  # (2, sum(2l+1))
        return np.concatenate([Y[:, o:o + 2 * l + 1].T.reshape(-1) for l, o in zip(ls, np.cumsum([0] + [2 * l + 1 for l in ls]))])[None, :]

    g, b, a = 0.9, 0.41, -2.3
    cases = [
        (descriptors.y_rotation(irreps), [encode(g, 4)], Ry(g)),
        (descriptors.x_rotation(irreps, 6), [encode(b, 6)], Rx(b)),
        (descriptors.xy_rotation(irreps), [encode(g, 4), encode(b, 4)], Rx(b) @ Ry(g)),
        (descriptors.yxy_rotation(irreps, 5), [encode(g, 5), encode(b, 5), encode(a, 5)], Ry(a) @ Rx(b) @ Ry(g)),
    ]
    axis = np.array([1.0, 2.0, -0.5]) / np.linalg.norm([1.0, 2.0, -0.5])
    K = np.array([[0, -axis[2], axis[1]], [axis[2], 0, -axis[0]], [-axis[1], axis[0], 0]])
    cases.append((descriptors.fixed_axis_angle_rotation(irreps, axis, 1.1), [], np.eye(3) + np.sin(1.1) * K + (1 - np.cos(1.1)) * K @ K))
    for e, enc, R in cases:
        assert np.allclose(evaluate(e, *enc, features(v)), features(v @ R.T), atol=1e-10)


def test_path_counts_and_operand_sizes_follow_the_construction_of_the_reference():
    """The reference builds the y rotation from one path for the middle component and four diagonal or anti-diagonal blocks of
    ``l`` entries per irrep (``rotations.py:150-187``): ``1 + 4 l`` scalar paths; the angle operand has ``2 lmax + 1`` elements."""
    irreps = cue.Irreps("O3", "2x0e+2x1o+2x2e+2x3o")
    e = descriptors.y_rotation(irreps)
    assert e.polynomial.operations[0][1].num_paths == sum(1 + 4 * ir.l for _, ir in irreps) == 28
    assert [o.size for o in e.polynomial.inputs] == [7, irreps.dim] and e.polynomial.outputs[0].size == irreps.dim
    e = descriptors.yxy_rotation(irreps, 5)
    assert [o.size for o in e.polynomial.inputs] == [11, 11, 11, irreps.dim]
    with pytest.raises(ValueError):
        descriptors.y_rotation(cue.Irreps("SU2", "1x1/2"))
    with pytest.raises(ValueError):
        descriptors.inversion(cue.Irreps("SO3", "1x1"))


def test_inversion_is_the_parity():
    irreps = cue.Irreps("O3", "2x0e+1x0o+2x1o+1x1e+2x2e")
    x = np.random.default_rng(2).normal(size=(3, irreps.dim))
    y = evaluate(descriptors.inversion(irreps), x)
    sign = np.concatenate([np.full(mul * ir.dim, float(ir.p)) for mul, ir in irreps])
    assert np.array_equal(y, x * sign)
    ls = [0, 1, 2, 3]
    nat = cue.Irreps("O3", [(1, cue.O3(l, (-1) ** l)) for l in ls])
    v = np.random.default_rng(3).normal(size=(4, 3))
    Y = descriptors.spherical_harmonics_values(cue.O3(1, -1), ls, v)
    assert np.allclose(evaluate(descriptors.inversion(nat), Y), descriptors.spherical_harmonics_values(cue.O3(1, -1), ls, -v), atol=1e-12)


@pytest.mark.gpu
@pytest.mark.parametrize("layout", [cue.ir_mul, cue.mul_ir])
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_rotation_and_inversion_modules(device, dtype, layout):
    """``cuet.Rotation`` / ``cuet.Inversion`` on the GPU against the descriptors evaluated by the oracle: one angle triple per
    row and one for all rows, mixed multiplicities, both layouts, gradients with respect to the features and the angles."""
    from cuequivariance_amd import cuet

    irreps = cue.Irreps("O3", "4x0e+2x1o+4x2e+2x1e")
    rot = cuet.Rotation(irreps, layout=layout, device=device)
    inv = cuet.Inversion(irreps, layout=layout, device=device)
    g = torch.Generator().manual_seed(4)
    Z = 19
    x = torch.randn(Z, irreps.dim, dtype=torch.float64, generator=g)
    angles = torch.randn(3, Z, dtype=torch.float64, generator=g)
    tol = 1e-12 if dtype == torch.float64 else 1e-5
    e = descriptors.yxy_rotation(irreps)
    spec = spec_from_polynomial(e.polynomial)
    for per_row in (True, False):
        ang = angles if per_row else angles[:, :1]
        xs = x.clone().requires_grad_(True)
        an = ang.clone().requires_grad_(True)
        x_ir_mul = change_layout(xs, irreps, True) if layout != cue.ir_mul else xs
        enc = [cuet.encode_rotation_angle(an[k], rot.lmax) for k in range(3)]
        ref = naive_segmented_polynomial(spec, [*enc, x_ir_mul])[0]
        ref = change_layout(ref, irreps, False) if layout != cue.ir_mul else ref
        cot = torch.randn(ref.shape, dtype=torch.float64, generator=g)
        ref_gx, ref_ga = torch.autograd.grad(ref, [xs, an], cot)
        xd = x.to(dtype).to(device).requires_grad_(True)
        ad = ang.to(dtype).to(device).requires_grad_(True)
        got = rot(ad[0], ad[1], ad[2], xd)
        assert got.dtype == dtype and got.shape == ref.shape
        scale = ref.abs().max().item()
        assert (got.detach().cpu().double() - ref.detach()).abs().max().item() <= tol * scale
        gx, ga = torch.autograd.grad(got, [xd, ad], cot.to(dtype).to(device))
        assert (gx.cpu().double() - ref_gx).abs().max().item() <= tol * ref_gx.abs().max().item()
        assert (ga.cpu().double() - ref_ga).abs().max().item() <= 10 * tol * ref_ga.abs().max().item()
    sign = torch.cat([torch.full((mul * ir.dim,), float(ir.p), dtype=torch.float64) for mul, ir in irreps])
    assert torch.equal(inv(x.to(dtype).to(device)).cpu(), (x * sign).to(dtype))
    # a rotation is orthogonal: the norm of every row is kept; gamma = beta = alpha = 0 is the identity
    xd = x.to(dtype).to(device)
    r = rot(angles[0].to(dtype).to(device), angles[1].to(dtype).to(device), angles[2].to(dtype).to(device), xd)
    assert torch.allclose(r.norm(dim=1), xd.norm(dim=1), rtol=10 * tol)
    zero = torch.zeros(1, dtype=dtype, device=device)
    assert (rot(zero, zero, zero, xd) - xd).abs().max().item() <= tol * x.abs().max().item()


def test_vector_to_euler_angles_points_the_y_axis_at_the_vector():
    from cuequivariance_amd import cuet

    v = torch.tensor([[0.3, -1.2, 0.8], [0.0, 2.0, 0.0], [0.0, -3.0, 0.0], [1.0, 0.0, 0.0], [-0.5, 0.1, -2.0]], dtype=torch.float64)
    beta, alpha = cuet.vector_to_euler_angles(v)
    for k in range(len(v)):
        assert np.allclose(Ry(alpha[k].item()) @ Rx(beta[k].item()) @ np.array([0.0, 1.0, 0.0]), (v[k] / v[k].norm()).numpy(), atol=1e-12)
    assert beta[1].item() == 0.0 and abs(beta[2].item() - np.pi) < 1e-15 and alpha[1].item() == 0.0 and alpha[2].item() == 0.0
    assert cuet.vector_to_euler_angles(torch.zeros(2, 4, 3))[0].shape == (2, 4)
    enc = cuet.encode_rotation_angle(torch.tensor([0.25, -1.0], dtype=torch.float64), 3)
    assert enc.shape == (2, 7) and np.allclose(enc[0].numpy(), encode(0.25, 3)[0]) and np.allclose(enc[1].numpy(), encode(-1.0, 3)[0])


def test_removed_names_refuse_with_their_replacement():
    """The four classes the reference keeps as stubs (``primitives/deprecated.py``): importable, not constructible."""
    from cuequivariance_amd import cuet

    for name in ("TensorProduct", "EquivariantTensorProduct", "SymmetricTensorProduct", "IWeightedSymmetricTensorProduct"):
        with pytest.raises(ImportError, match="SegmentedPolynomial"):
            getattr(cuet, name)(None)


def test_composition_of_descriptors_by_dot():
    """``cue.segmented_polynomials.dot`` as the reference uses it to build its rotations (``rotations.py:70-77,94-96``): the y
    rotation composed with the x rotation over the intermediate features, operands moved into the order ``gamma, beta, input,
    output``, evaluates like ``xy_rotation``; with no pair given ``dot`` is the plain product of two descriptors."""
    irreps = cue.Irreps("O3", "2x0e+2x1o+2x2e")
    y = descriptors.y_rotation(irreps).polynomial.operations[0][1]   # gamma, input, A
    x = descriptors.x_rotation(irreps).polynomial.operations[0][1]   # beta, A, output
    d = cue.segmented_polynomials.dot(y, x, (2, 1)).move_operand(1, 2)  # gamma, input, beta, output -> gamma, beta, input, output
    assert d.subscripts == ",,u,u" and d.num_operands == 4
    g, b = 0.7, -0.4
    feats = np.random.default_rng(6).normal(size=(3, irreps.dim))
    got = naive_segmented_polynomial(spec_from_polynomial(cue.SegmentedPolynomial.eval_last_operand(d)),
                                     [torch.as_tensor(encode(g, 2)), torch.as_tensor(encode(b, 2)), torch.as_tensor(feats)])[0].numpy()
    assert np.allclose(got, evaluate(descriptors.xy_rotation(irreps), encode(g, 2), encode(b, 2), feats), atol=1e-12)
    a = cue.SegmentedTensorProduct.from_subscripts("i,j+ij")
    a.add_path(None, None, c=np.arange(6.0).reshape(2, 3))
    p = cue.segmented_polynomials.dot(a, a)
    assert p.num_operands == 4 and p.num_paths == 1 and p.coefficient_subscripts == "ij"
    with pytest.raises(ValueError):
        cue.segmented_polynomials.dot(y, x, (0, 1))
    assert hasattr(cue.group_theory, "clebsch_gordan") and cue.group_theory.descriptors is descriptors


@pytest.mark.gpu
def test_rotation_traced_as_a_whole(device):
    """``torch.compile(fullgraph=True)`` and ``torch.export`` of ``cuet.Rotation`` (angle encodings in torch code, the polynomial
    through the opaque uniform-1d operator) against the eager module."""
    from cuequivariance_amd import cuet

    irreps = cue.Irreps("O3", "4x0e+4x1o+4x2e")
    rot = cuet.Rotation(irreps, layout=cue.ir_mul, device=device)
    g = torch.Generator(device=device).manual_seed(7)
    x = torch.randn(11, irreps.dim, device=device, generator=g)
    a = torch.randn(3, 11, device=device, generator=g)
    want = rot(a[0], a[1], a[2], x)
    got = torch.compile(rot, fullgraph=True)(a[0], a[1], a[2], x)
    assert (got - want).abs().max().item() <= 1e-6 * want.abs().max().item()
    program = torch.export.export(rot, (a[0].clone(), a[1].clone(), a[2].clone(), x.clone()))
    out = program.module()(a[0], a[1], a[2], x)
    assert (out - want).abs().max().item() <= 1e-6 * want.abs().max().item()
