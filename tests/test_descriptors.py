"""Pins the descriptor compiler: segmented tensor products, their transforms, polynomials, tables.

Known answers are taken from the reference's own tests and doc examples:

* ``cuequivariance/tests/segmented_polynomials/segmented_tensor_product_test.py`` (string forms :26-63,
  squeeze :66-86, normalisation :89-112, flatten invariance :134-154, consolidate_paths :205-218,
  serialisation :221-236, exact ``to_text`` dump :239-259, split_mode :276-344)
* ``.../operation_test.py:18-63`` and ``.../segmented_polynomial_test.py:171-270`` (jvp / transpose / backward)
* doc examples: fully connected "61440 weights, 15 paths" (``descriptors/irreps_tp.py:72-78``), flattened text
  (``segmented_tensor_product.py:335-356``), path counts 4/12/11 (``equivariant_polynomial.py:435-442``).
"""

import numpy as np
import pytest

from cuequivariance_amd import cue
from cuequivariance_amd.tables import U1dTables


def make_coeffs(shape):
    return (np.arange(np.prod(shape)) + 1.0).reshape(shape)


def test_user_friendly_strings():
    d = cue.SegmentedTensorProduct.from_subscripts("ia_jb_kab+ijk")
    assert str(d) == "ia,jb,kab+ijk sizes=0,0,0 num_segments=0,0,0 num_paths=0 a= b= i= j= k="
    with pytest.raises(ValueError):
        d.add_path(0, 0, 0, c=make_coeffs((2, 2, 3)))
    with pytest.raises(ValueError):
        d.add_segment(0, (2, 2, 2))
    d.add_segment(0, (5, 16))
    d.add_segment(1, (5, 32))
    d.add_segment(2, (4, 16, 32))
    d.add_segment(2, (4, 32, 32))
    with pytest.raises(ValueError):
        d.add_path(0, 0, 0, c=make_coeffs((5, 5, 5)))
    assert str(d) == "ia,jb,kab+ijk sizes=80,160,6144 num_segments=1,1,2 num_paths=0 a={16, 32} b=32 i=5 j=5 k=4"
    d.add_path(0, 0, 0, c=make_coeffs((5, 5, 4)))
    assert d.num_paths == 1 and not d.all_segments_are_used()
    assert d.subscripts == "ia,jb,kab+ijk"
    d.assert_valid()


def test_squeeze():
    d = cue.SegmentedTensorProduct.from_subscripts("i_j+ij")
    d.add_segment(0, (1,))
    d.add_segment(1, (20,))
    d.add_path(0, 0, c=make_coeffs((1, 20)))
    assert d.squeeze_modes().subscripts == ",j+j"
    d = cue.SegmentedTensorProduct.from_subscripts("i_j+ij")
    d.add_segment(0, (1,))
    d.add_segment(0, (2,))
    d.add_segment(1, (20,))
    d.add_path(0, 0, c=make_coeffs((1, 20)))
    d.add_path(1, 0, c=make_coeffs((2, 20)))
    assert d.squeeze_modes().subscripts == "i,j+ij"
    with pytest.raises(ValueError):
        d.squeeze_modes("i")


def test_normalize_paths_for_operand():
    d = cue.SegmentedTensorProduct.from_subscripts("i_j+ij")
    d.add_segments(0, 2 * [(2,)])
    d.add_segments(1, 2 * [(3,)])
    d.add_path(0, 0, c=np.array([[2, 0, 0], [0, 2, 0]]))
    d = d.normalize_paths_for_operand(0)
    np.testing.assert_allclose(d.paths[0].coefficients, np.array([[1, 0, 0], [0, 1, 0]]))


def make_example_descriptor(rng):
    d = cue.SegmentedTensorProduct.from_subscripts("uv_iu_jv+ij")
    d.add_path(None, None, None, c=rng.normal(size=(2, 3)), dims={"u": 4, "v": 5, "i": 2, "j": 3})
    d.add_path(None, None, None, c=rng.normal(size=(4, 5)), dims={"u": 2, "v": 3, "i": 4, "j": 5})
    d.assert_valid()
    return d


def test_flatten_preserves_evaluation():
    rng = np.random.default_rng(1)
    d = make_example_descriptor(rng)
    assert d.flatten_modes("").subscripts == "uv,iu,jv+ij"
    assert d.flatten_modes("i").subscripts == "uv,u,jv+j"
    assert d.flatten_modes("j").subscripts == "uv,iu,v+i"
    assert d.flatten_modes("ij").subscripts == "uv,u,v"
    assert d.flatten_modes("ui").subscripts == "v,,jv+j"
    assert d.flatten_coefficient_modes().subscripts == "uv,u,v"
    x0, x1 = rng.normal(size=d.operands[0].size), rng.normal(size=d.operands[1].size)
    ref = d.compute_last_operand(x0, x1)
    for modes in ["i", "j", "ij", "ui", "iju", "uvij"]:
        np.testing.assert_allclose(ref, d.flatten_modes(modes).compute_last_operand(x0, x1), atol=1e-12)


def test_flattened_text_dump_exact():
    d = cue.SegmentedTensorProduct.from_subscripts("iu,ju,ku+ijk")
    d.add_path(None, None, None, c=make_coeffs((3, 3, 3)), dims={"u": 12})
    d.add_path(None, None, None, c=make_coeffs((1, 2, 1)), dims={"u": 14})
    d = d.flatten_modes("ijk")
    expected = """u,u,u sizes=50,64,50 num_segments=4,5,4 num_paths=29 u={12, 14}
operand #0 subscripts=u
  | u: [12, 12, 12, 14]
operand #1 subscripts=u
  | u: [12, 12, 12, 14, 14]
operand #2 subscripts=u
  | u: [12, 12, 12, 14]
Memory cost: 164
Path indices: 0 0 0, 0 0 1, 0 0 2, 0 1 0, 0 1 1, 0 1 2, 0 2 0, 0 2 1, 0 2 2, 1 0 0, 1 0 1, 1 0 2, 1 1 0, 1 1 1, 1 1 2, 1 2 0, 1 2 1, 1 2 2, 2 0 0, 2 0 1, 2 0 2, 2 1 0, 2 1 1, 2 1 2, 2 2 0, 2 2 1, 2 2 2, 3 3 3, 3 4 3
Path coefficients: [1.0 2.0 3.0 4.0 5.0 6.0 7.0 8.0 9.0 10.0 11.0 12.0 13.0 14.0 15.0 16.0 17.0 18.0 19.0 20.0 21.0 22.0 23.0 24.0 25.0 26.0 27.0 1.0 2.0]"""
    assert d.to_text() == expected  # the reference's dump minus its "Flop cost" line


def test_fully_connected_doc_examples():
    e = cue.descriptors.fully_connected_tensor_product(
        16 * cue.Irreps("SO3", "0 + 1 + 2"), 16 * cue.Irreps("SO3", "0 + 1 + 2"), 16 * cue.Irreps("SO3", "0 + 1 + 2")
    )
    (_, d), = e.polynomial.operations
    assert e.inputs[0].dim == 61440 and d.num_paths == 15 and d.subscripts == "uvw,iu,jv,kw+ijk"
    (_, d), = cue.descriptors.fully_connected_tensor_product(
        cue.Irreps("SO3", "4x0+4x1"), cue.Irreps("SO3", "4x0+4x1"), cue.Irreps("SO3", "4x0+4x1")
    ).polynomial.operations
    d = d.flatten_coefficient_modes()
    assert str(d) == "uvw,u,v,w sizes=320,16,16,16 num_segments=5,4,4,4 num_paths=16 u=4 v=4 w=4"
    assert [tuple(p.indices) for p in d.paths[:6]] == [
        (0, 0, 0, 0), (1, 0, 1, 1), (1, 0, 2, 2), (1, 0, 3, 3), (2, 1, 0, 1), (2, 2, 0, 2)
    ]
    # normalisation: cg / sqrt(sum over paths into the segment of mean(c^2) * u * v * i * j)
    assert f"{float(d.paths[0].coefficients):.2f}" == "0.18" or f"{float(d.paths[0].coefficients):.2f}" == "0.17"
    assert 0.17 <= float(d.paths[0].coefficients) < 0.18


def test_channelwise_counts_and_order():
    e = cue.descriptors.channelwise_tensor_product(
        cue.Irreps("SO3", "64x0 + 32x1"), cue.Irreps("SO3", "0 + 1"), simplify_irreps3=True
    )
    assert repr(e.outputs[0].irreps) == "96x0+128x1+32x2" and e.inputs[0].dim == 256
    # reference doc: paths per output irrep 4 / 12 / 11  => nnz(CG) of 000,011,101,110,111,112 = 1,3,3,3,6,11
    nnz = {}
    for l1, l2, l3 in [(0, 0, 0), (0, 1, 1), (1, 0, 1), (1, 1, 0), (1, 1, 1), (1, 1, 2)]:
        nnz[(l1, l2, l3)] = np.count_nonzero(cue.SO3.clebsch_gordan(cue.SO3(l1), cue.SO3(l2), cue.SO3(l3)))
    assert nnz == {(0, 0, 0): 1, (0, 1, 1): 3, (1, 0, 1): 3, (1, 1, 0): 3, (1, 1, 1): 6, (1, 1, 2): 11}
    assert e.polynomial.operations[0][1].num_paths == 4 + 12 + 11

    e = cue.descriptors.channelwise_tensor_product(
        cue.Irreps("O3", "128x0e+128x1o+128x2e+128x3o"), cue.Irreps("O3", "0e+1o+2e+3o"), "0e+1o+2e+3o"
    )
    d = e.polynomial.operations[0][1]
    assert d.subscripts == "uv,iu,jv,kuv+ijk" and d.num_paths == 23
    assert [o.size for o in d.operands] == [2944, 2048, 16, 12672]
    assert [m for m, _ in e.outputs[0].irreps] == [128] * 23
    assert [repr(ir) for _, ir in e.outputs[0].irreps] == ["0e"] * 4 + ["1o"] * 6 + ["2e"] * 7 + ["3o"] * 6
    # channel-wise coefficients are left untouched by the normalisation (one path per output segment)
    for p in d.paths:
        assert abs((p.coefficients**2).sum() - p.coefficients.shape[2]) < 1e-10
    # generation order is (i1 major, i2, l3 ascending); sorting renumbers segments, paths keep their order
    assert [p.indices[1:3] for p in d.paths[:4]] == [(0, 0), (0, 1), (0, 2), (0, 3)]
    assert d.paths[1].indices == (4, 0, 1, 4)  # 0e x 1o -> first 1o segment, which sits after the four 0e
    f = e.polynomial.flatten_coefficient_modes().squeeze_modes().operations[0][1]
    assert f.subscripts == "u,u,,u" and [len(o) for o in f.operands] == [23, 16, 16, 99]

    e = cue.descriptors.channelwise_tensor_product(
        cue.Irreps("O3", "32x0e+32x1o+32x2e"), cue.Irreps("O3", "0e+1o+2e"), "0e+1o+2e"
    )
    assert [o.size for o in e.polynomial.operands] == [352, 288, 9, 1120]


def test_linear_normalisation():
    e = cue.descriptors.linear(cue.Irreps("O3", "128x0e+128x1o+128x2e"), cue.Irreps("O3", "128x0e+128x1o+128x2e"))
    d = e.polynomial.operations[0][1]
    assert d.subscripts == "uv,iu,iv" and d.num_paths == 3 and e.inputs[0].dim == 49152
    for p in d.paths:
        assert abs(float(p.coefficients) - 1 / np.sqrt(128)) < 1e-15


def test_squeeze_flatten_commute():
    i1, i2, i3 = cue.Irreps("O3", "32x0e + 32x1o"), cue.Irreps("O3", "1x0e + 1x1o"), cue.Irreps("O3", "32x0e + 32x1o")
    for e in [
        cue.descriptors.fully_connected_tensor_product(i1, i2, i3),
        cue.descriptors.channelwise_tensor_product(i1, i2, i3),
        cue.descriptors.linear(i1, i3),
    ]:
        a = e.polynomial.squeeze_modes().flatten_coefficient_modes()
        b = e.polynomial.flatten_coefficient_modes().squeeze_modes()
        assert a == b


def test_serialisation_roundtrip_and_hash():
    d = cue.SegmentedTensorProduct.from_subscripts("ui,uj,uk+ijk")
    d.add_path(None, None, None, c=make_coeffs((3, 3, 3)), dims={"u": 12})
    d.add_path(None, None, None, c=make_coeffs((1, 2, 1)), dims={"u": 14})
    assert d == cue.SegmentedTensorProduct.from_dict(d.to_dict())
    assert d == cue.SegmentedTensorProduct.from_json(d.to_json())
    assert d == cue.SegmentedTensorProduct.from_base64(d.to_base64())
    d2 = cue.SegmentedTensorProduct.from_subscripts("ui,uj,uk+ijk")
    assert hash(d) != hash(d2)
    d2.add_path(None, None, None, c=make_coeffs((3, 3, 3)), dims={"u": 12})
    d2.add_path(None, None, None, c=make_coeffs((1, 2, 1)), dims={"u": 14})
    assert hash(d) == hash(d2) and d == d2


def test_consolidate_paths_and_split_mode():
    d = cue.SegmentedTensorProduct.from_subscripts("ab_ab+ab")
    d.add_segment(0, (2, 3))
    d.add_segment(1, (2, 3))
    d.add_path(0, 0, c=make_coeffs((2, 3)))
    d.add_path(0, 0, c=make_coeffs((2, 3)))
    np.testing.assert_allclose(d.consolidate_paths().stacked_coefficients, 2 * make_coeffs((1, 2, 3)))

    d = cue.SegmentedTensorProduct.from_subscripts("ua,ub+ab")
    d.add_segment(0, (6, 4))
    d.add_segment(1, (6, 5))
    d.add_path(0, 0, c=make_coeffs((4, 5)))
    s2 = d.split_mode("u", 2)
    assert s2.operands[0].num_segments == 3 and s2.operands[1].num_segments == 3 and s2.subscripts == "ua,ub+ab"
    assert all(seg == (2, 4) for seg in s2.operands[0]) and all(seg == (2, 5) for seg in s2.operands[1])
    assert d.split_mode("u", 3).operands[0].num_segments == 2
    with pytest.raises(ValueError):
        d.split_mode("u", 5)
    assert d.split_mode("v", 2) == d
    dc = cue.SegmentedTensorProduct.from_subscripts("au,bu+ab")
    dc.add_segment(0, (3, 6))
    dc.add_segment(1, (4, 6))
    dc.add_path(0, 0, c=make_coeffs((3, 4)))
    with pytest.raises(ValueError):
        dc.split_mode("u", 2)
    # evaluation is preserved by splitting
    d3 = cue.SegmentedTensorProduct.from_subscripts("ua,ub,uc+abc")
    d3.add_path(None, None, None, c=make_coeffs((2, 3, 2)), dims={"u": 6})
    rng = np.random.default_rng(0)
    x0, x1 = rng.normal(size=12), rng.normal(size=18)
    np.testing.assert_allclose(d3.compute_last_operand(x0, x1), d3.split_mode("u", 2).compute_last_operand(x0, x1))


def test_evaluate_matmul_identities():
    rng = np.random.default_rng(2)
    d = cue.SegmentedTensorProduct.from_subscripts("uv_vw_uw")
    d.add_path(None, None, None, c=1.0, dims={"u": 2, "v": 3, "w": 4})
    x0, x1 = rng.normal(size=(10, 6)), rng.normal(size=(10, 12))
    np.testing.assert_allclose(
        d.compute_last_operand(x0, x1), (x0.reshape(10, 2, 3) @ x1.reshape(10, 3, 4)).reshape(10, -1)
    )
    d = cue.SegmentedTensorProduct.from_subscripts("iuv_jvw_kuw+ijk")
    c = rng.normal(size=(2, 3, 4))
    d.add_path(None, None, None, c=c, dims={"u": 2, "v": 3, "w": 4})
    x0, x1 = rng.normal(size=d.operands[0].size), rng.normal(size=d.operands[1].size)
    ref = np.einsum("ijk,iuv,jvw->kuw", c, x0.reshape(2, 2, 3), x1.reshape(3, 3, 4)).reshape(-1)
    np.testing.assert_allclose(d.compute_last_operand(x0, x1), ref)


# ------------------------------------------------------------------------------ operations / polynomials
def test_operation_transpose_and_jvp():
    ope = cue.Operation([0, 1, 2, 3])
    assert ope.transpose([True, False, False], [True]) == cue.Operation([3, 0, 1, 2])
    assert cue.Operation([0, 1, 2, 4]).transpose([True, False, False, True], [True]) == cue.Operation([3, 0, 1, 2])
    assert cue.Operation([4, 2, 3, 1]).transpose([True, False, False, True], [True]) == cue.Operation([2, 1, 4, 0])
    cube = cue.Operation([0, 0, 0, 1])
    assert cube.jvp([True]) == [cue.Operation((1, 0, 0, 2)), cue.Operation((0, 1, 0, 2)), cue.Operation((0, 0, 1, 2))]
    assert cue.Operation((0, 0, 1, 2)).transpose([False, True], [True]) == cue.Operation((0, 0, 2, 1))
    with pytest.raises(ValueError):
        cue.Operation((0, 0, 1)).transpose([True], [True])


def dot_product_stp():
    d = cue.SegmentedTensorProduct.from_subscripts("i,j,k+ijk")
    d.add_path(d.add_segment(0, (3,)), d.add_segment(1, (3,)), d.add_segment(2, (1,)), c=np.eye(3).reshape(3, 3, 1))
    return d


def test_polynomial_jvp_transpose_backward_closed_forms():
    poly = cue.SegmentedPolynomial.eval_last_operand(dot_product_stp())
    x, y = np.array([1.0, 2.0, 3.0]), np.array([4.0, 5.0, 6.0])
    xt, yt = np.array([0.1, 0.2, 0.3]), np.array([0.4, 0.5, 0.6])
    np.testing.assert_allclose(poly(x, y)[0], [x.dot(y)])
    jvp, m = poly.jvp([True, True])
    assert m(([0, 1], [2])) == ([0, 1, 0, 1], [2])
    np.testing.assert_allclose(jvp(x, y, xt, yt)[0], [y.dot(xt) + x.dot(yt)])
    np.testing.assert_allclose(poly.jvp([True, False])[0](x, y, xt)[0], [y.dot(xt)])
    np.testing.assert_allclose(poly.jvp([False, True])[0](x, y, yt)[0], [x.dot(yt)])
    cot = np.array([2.0])
    np.testing.assert_allclose(poly.transpose([True, False], [True])[0](y, cot)[0], 2 * y)
    np.testing.assert_allclose(poly.transpose([False, True], [True])[0](x, cot)[0], 2 * x)
    gx, gy = poly.backward([True, True], [True])[0](x, y, cot)
    np.testing.assert_allclose(gx, 2 * y)
    np.testing.assert_allclose(gy, 2 * x)
    [gx] = poly.backward([True, False], [True])[0](x, y, cot)
    np.testing.assert_allclose(gx, 2 * y)


def test_jvp_of_repeated_operand_has_multiplicity():
    # f(x) = sum_i x_i^3 through a degree-3 operation on one buffer
    d = cue.SegmentedTensorProduct.empty_segments([2, 2, 2, 1])
    d.add_path(0, 0, 0, 0, c=1.0)
    d.add_path(1, 1, 1, 0, c=1.0)
    poly = cue.SegmentedPolynomial([d.operands[0]], [d.operands[-1]], [(cue.Operation([0, 0, 0, 1]), d)])
    x, t = np.array([2.0, -3.0]), np.array([0.5, 0.25])
    np.testing.assert_allclose(poly(x)[0], [(x**3).sum()])
    jvp, _ = poly.jvp([True])
    assert len(jvp.operations) == 1  # the three slots are merged into one operation with weight 3
    np.testing.assert_allclose(jvp(x, t)[0], [(3 * x**2 * t).sum()])
    bwd, _ = poly.backward([True], [True])
    np.testing.assert_allclose(bwd(x, np.array([1.0]))[0], 3 * x**2)


def test_channelwise_polynomial_backward_matches_finite_differences():
    e = cue.descriptors.channelwise_tensor_product(cue.Irreps("O3", "2x0e+2x1o"), cue.Irreps("O3", "0e+1o"), "0e+1o")
    poly = e.polynomial.flatten_coefficient_modes().squeeze_modes()
    rng = np.random.default_rng(3)
    w, x1, x2 = (rng.normal(size=o.size) for o in poly.inputs)
    g = rng.normal(size=poly.outputs[0].size)
    bwd, _ = poly.backward([True, True, True], [True])
    gw, gx1, gx2 = bwd(w, x1, x2, g)

    def f(w, x1, x2):
        return float(poly(w, x1, x2)[0] @ g)

    h = 1e-6
    for grad, k in [(gw, 0), (gx1, 1), (gx2, 2)]:
        args = [w, x1, x2]
        num = np.zeros_like(args[k])
        for i in range(args[k].size):
            a, b = [v.copy() for v in args], [v.copy() for v in args]
            a[k][i] += h
            b[k][i] -= h
            num[i] = (f(*a) - f(*b)) / (2 * h)
        np.testing.assert_allclose(grad, num, atol=1e-6)


# ------------------------------------------------------------------------------ flat tables
def test_uniform1d_tables_by_hand():
    # out[0] = 2 a[0] b[1] ; out[1] = -3 a[1] b[0] * scalar s[0]; a, b, out are u-vectors (u=4), s scalar
    d = cue.SegmentedTensorProduct.from_subscripts("u,u,,u")
    d.add_segments(0, [(4,), (4,)])
    d.add_segments(1, [(4,), (4,)])
    d.add_segments(2, [()])
    d.add_segments(3, [(4,), (4,)])
    d.add_path(0, 1, 0, 0, c=2.0)
    d.add_path(1, 0, 0, 1, c=-3.0)
    t = U1dTables.from_polynomial(cue.SegmentedPolynomial.eval_last_operand(d))
    assert t.operand_extent == 4 and (t.num_inputs, t.num_outputs) == (3, 1)
    assert t.buffer_dim == (1, 1, 0, 1) and t.buffer_num_segments == (2, 2, 1, 2)
    assert t.dtypes == (0, 1, 2, 0)
    assert t.num_operands == (4,) and t.operations == (0, 1, 2, 3) and t.num_paths == (2,)
    assert t.path_indices_start == (0,) and t.path_coefficients_start == (0,)
    assert t.path_indices == (0, 1, 0, 0, 1, 0, 0, 1) and t.path_coefficients == (2.0, -3.0)
    b = t.backward((True, False, True))
    assert (b.num_inputs, b.num_outputs) == (4, 2)
    assert b.operations == (4, 1, 2, 3, 0, 1, 5, 3)  # d a reads cotangent (buffer 3), writes buffer 4; d s writes 5
    assert b.buffer_dim == (1, 1, 0, 1, 1, 0) and b.buffer_num_segments == (2, 2, 1, 2, 2, 1)
    assert b.path_indices_start == (0, 0) and b.path_indices == t.path_indices
    assert b.dtypes == (0, 1, 2, 3, 0, 2)


def test_cfg2_tables():
    e = cue.descriptors.channelwise_tensor_product(
        cue.Irreps("O3", "128x0e+128x1o+128x2e+128x3o"), cue.Irreps("O3", "0e+1o+2e+3o"), "0e+1o+2e+3o"
    )
    t = U1dTables.from_polynomial(e.polynomial.flatten_coefficient_modes().squeeze_modes())
    assert t.operand_extent == 128 and t.buffer_dim == (1, 1, 0, 1) and t.buffer_num_segments == (23, 16, 16, 99)
    assert t.num_paths == (353,) and len(t.path_indices) == 4 * 353
    # first block is 0e x 0e -> 0e with coefficient 1, then 0e x 1o -> 1o: three paths with coefficient 1
    assert t.path_indices[:16] == (0, 0, 0, 0, 4, 0, 1, 4, 4, 0, 2, 5, 4, 0, 3, 6)
    np.testing.assert_allclose(t.path_coefficients[:4], [1.0, 1.0, 1.0, 1.0], atol=1e-12)
    # element offset of segment s of buffer b in a row is s * extent (or s for scalars)
    assert t.width(0) == 2944 and t.width(1) == 2048 and t.width(2) == 16 and t.width(3) == 12672


def test_spherical_harmonics_polynomial():
    """Path counts of the doc example (``descriptors/spherical_harmonics_.py:70-76``), the value at (0, 1, 0)
    (``cuequivariance_jax/segmented_polynomials/segmented_polynomial.py:112-117``), the norm on unit vectors and agreement
    with the independent value recursion."""
    e = cue.descriptors.spherical_harmonics(cue.SO3(1), [0, 1, 2])
    assert [d.num_paths for _, d in e.polynomial.operations] == [1, 3, 11]
    [y] = e.polynomial(np.array([0.0, 1.0, 0.0]))
    np.testing.assert_allclose(y, [1, 0, np.sqrt(3), 0, 0, 0, np.sqrt(5), 0, 0], atol=1e-14)
    ls = [0, 1, 2, 3, 4]
    p = cue.descriptors.spherical_harmonics(cue.O3(1, -1), ls).polynomial
    x = np.random.default_rng(0).normal(size=(7, 3))
    x /= np.linalg.norm(x, axis=1, keepdims=True)
    [y] = p(x)
    np.testing.assert_allclose(y, cue.descriptors.spherical_harmonics_values(cue.O3(1, -1), ls, x), atol=1e-13)
    off = 0
    for ell in ls:
        np.testing.assert_allclose((y[:, off: off + 2 * ell + 1] ** 2).sum(1), 2 * ell + 1, atol=1e-12)
        off += 2 * ell + 1


def test_weightless_products_and_the_transpose_descriptor():
    """``full_tensor_product`` is the channel-wise product with every weight one (that descriptor is pinned to the reference's
    expectations above); ``elementwise_tensor_product`` is its diagonal in the two channel indices, with the multiplicities of
    the two operands cut to match; ``transpose`` moves every element between the two layouts.  Evaluated by the oracle."""
    import torch

    from oracle.naive import naive_segmented_polynomial, spec_from_polynomial

    def run(e, *xs):
        return naive_segmented_polynomial(spec_from_polynomial(e.polynomial), [torch.as_tensor(x) for x in xs])[0].numpy()

    rng = np.random.default_rng(5)
    a, b = cue.Irreps("O3", "2x0e+3x1o+1x2e"), cue.Irreps("O3", "1x0e+2x1o")
    full = cue.descriptors.full_tensor_product(a, b, ["0e", "1o", "2e"])
    cw = cue.descriptors.channelwise_tensor_product(a, b, ["0e", "1o", "2e"])
    assert full.outputs[0].irreps == cw.outputs[0].irreps and full.polynomial.operations[0][1].subscripts == "iu,jv,kuv+ijk"
    x1, x2 = rng.normal(size=(4, a.dim)), rng.normal(size=(4, b.dim))
    assert np.allclose(run(full, x1, x2), run(cw, np.ones((4, cw.inputs[0].irreps.dim)), x1, x2), atol=1e-13)

    c, d = cue.Irreps("O3", "3x1o+4x0e"), cue.Irreps("O3", "3x1o+2x0e+2x0o")
    el = cue.descriptors.elementwise_tensor_product(c, d)
    assert str(el.inputs[0].irreps) == "3x1o+2x0e+2x0e" and str(el.inputs[1].irreps) == "3x1o+2x0e+2x0o"
    assert str(el.outputs[0].irreps) == "3x0e+3x1e+3x2e+2x0e+2x0o" and el.polynomial.operations[0][1].subscripts == "iu,ju,ku+ijk"
    y1, y2 = rng.normal(size=(2, c.dim)), rng.normal(size=(2, d.dim))
    got = run(el, y1, y2)
    # the first three output irreps against the diagonal of the full product of 3x1o with 3x1o (ir_mul rows: (component, u, v))
    f = run(cue.descriptors.full_tensor_product(cue.Irreps("O3", "3x1o"), cue.Irreps("O3", "3x1o")), y1[:, :9], y2[:, :9])
    off_f = off_g = 0
    for dim in (1, 3, 5):
        block = f[:, off_f:off_f + dim * 9].reshape(2, dim, 3, 3)
        assert np.allclose(got[:, off_g:off_g + dim * 3].reshape(2, dim, 3), np.einsum("zkuu->zku", block), atol=1e-13)
        off_f, off_g = off_f + dim * 9, off_g + dim * 3
    assert np.allclose(got[:, off_g:off_g + 2], y1[:, 9:11] * y2[:, 9:11]) and np.allclose(got[:, off_g + 2:], y1[:, 11:13] * y2[:, 11:13])
    with pytest.raises(ValueError):
        cue.descriptors.elementwise_tensor_product(cue.Irreps("O3", "2x0e"), cue.Irreps("O3", "1x0e+2x1o"))

    t = cue.descriptors.transpose(a, cue.mul_ir, cue.ir_mul)
    z = rng.normal(size=(3, a.dim))
    want = np.concatenate([z[:, o:o + m * ir.dim].reshape(3, m, ir.dim).transpose(0, 2, 1).reshape(3, -1)
                           for (m, ir), o in zip(a, np.cumsum([0] + [m * ir.dim for m, ir in a]))], axis=1)
    assert np.array_equal(run(t, z), want)
    assert np.array_equal(run(cue.descriptors.transpose(a, cue.ir_mul, cue.mul_ir), want), z)


def test_assumed_irrep_class_and_layout():
    """``cue.assume`` as context manager and decorator (reference ``irreps_array/context_decorator.py:33-84``): the irrep class of
    ``cue.Irreps("2x1")`` and the layout of ``cue.IrrepsAndLayout`` without one; scopes nest and are restored."""
    with pytest.raises(ValueError):
        cue.get_irrep_scope()
    assert cue.get_irrep_scope(raising=False) is None and cue.get_layout_scope(raising=False) is None
    with cue.assume(cue.SO3, cue.mul_ir):
        rep = cue.IrrepsAndLayout("2x1")
        assert rep.irreps == cue.Irreps("SO3", "2x1") and rep.layout == cue.mul_ir
        with cue.assume("O3", cue.ir_mul):
            assert cue.Irreps("2x1o").irrep_class is cue.O3 and cue.IrrepsAndLayout("1e").layout == cue.ir_mul
            assert cue.get_irrep_scope() is cue.O3 and cue.get_layout_scope() == cue.ir_mul
        assert cue.get_irrep_scope() is cue.SO3 and cue.get_layout_scope() == cue.mul_ir
    assert cue.get_irrep_scope(raising=False) is None

    @cue.assume(cue.SU2)
    def half():
        return cue.Irreps("3x1/2")

    assert half().irrep_class is cue.SU2
    with cue.assume(cue.ir_mul):  # a layout alone
        assert cue.get_layout_scope() == cue.ir_mul and cue.get_irrep_scope(raising=False) is None
