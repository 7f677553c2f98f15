"""The names the reference's torch frontend imports from its closed operator package, served by this engine
(``cuequivariance_amd.ops_torch``): registration and schema on the CPU, results on the GPU."""

import numpy as np
import pytest
import torch

from cuequivariance_amd import cue
from cuequivariance_amd.tables import U1dTables
from oracle.naive import naive_segmented_polynomial, spec_from_polynomial


def rel_err(got, ref):
    got, ref = got.detach().cpu().double(), ref.detach().cpu().double()
    return (got - ref).abs().max().item() / max(ref.abs().max().item(), 1e-30)


def channelwise_poly():
    e = cue.descriptors.channelwise_tensor_product(
        cue.Irreps("O3", "8x0e+8x1o"), cue.Irreps("O3", "0e+1o"), ["0e", "1o"], True)
    return e.polynomial


def test_registration_and_schema():
    """``register_ops`` defines ``torch.ops.cuequivariance.uniform_1d`` with the 21 arguments of the reference's call
    (``cuequivariance_torch/primitives/segmented_polynomial_uniform_1d.py:32-77``), and is idempotent."""
    from cuequivariance_amd import ops_torch

    ops_torch.register_ops()
    ops_torch.register_ops()
    schema = torch.ops.cuequivariance.uniform_1d.default._schema
    names = [a.name for a in schema.arguments]
    assert names == ["name", "math_dtype", "operand_extent", "num_inputs", "num_outputs", "num_index", "buffer_dim",
                     "buffer_num_segments", "batch_dim", "index_buffer", "dtypes", "num_operations", "num_operands",
                     "operations", "num_paths", "path_indices_start", "path_coefficients_start", "path_indices",
                     "path_coefficients", "batch_size", "tensors"]
    assert str(schema.returns[0].type) == "List[Tensor]"
    c = ops_torch.uniform_1d
    assert len({c.BATCH_DIM_AUTO, c.BATCH_DIM_SHARED, c.BATCH_DIM_BATCHED, c.BATCH_DIM_INDEXED}) == 4
    assert [p.name for p in ops_torch.TriMulPrecision] == ["NONE", "DEFAULT", "TF32", "TF32x3", "IEEE"]
    assert [p.value for p in ops_torch.TriMulPrecision] == [-1, 0, 1, 2, 3]


def test_uniform_1d_plan_lookup_by_argument_values(monkeypatch):
    """``uniform_1d`` finds its plan by the values of the lists it is given: equal lists (other objects) meet the same
    plan, a changed coefficient or another arithmetic type meets another one."""
    import importlib

    u = importlib.import_module("cuequivariance_amd.cuet.uniform_1d")
    seen = []
    monkeypatch.setattr(u, "run_plan", lambda plan, *a, **k: seen.append(plan) or [])
    t = U1dTables.from_polynomial(channelwise_poly().flatten_coefficient_modes().squeeze_modes())

    def call(coefficients, math_dtype=torch.float32):
        return u.uniform_1d(
            "lookup", math_dtype, t.operand_extent, t.num_inputs, t.num_outputs, 0, list(t.buffer_dim), list(t.buffer_num_segments),
            [0] * 4, [-1] * 4, list(t.dtypes), len(t.num_operands), list(t.num_operands), list(t.operations), list(t.num_paths),
            list(t.path_indices_start), list(t.path_coefficients_start), list(t.path_indices), coefficients, 0, [])

    c = list(t.path_coefficients)
    call(c), call(list(c)), call([2.0 * c[0]] + c[1:]), call(c, torch.float64)
    assert seen[0] is seen[1]
    assert seen[2] is not seen[0] and seen[2].tables.path_coefficients[0] == 2.0 * c[0]
    assert seen[3] is not seen[0] and seen[3].math_dtype == torch.float64


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_uniform_1d_through_torch_ops(device, dtype):
    """The frontend's call, literally: lists built the way ``segmented_polynomial_uniform_1d.py:188-292`` builds them,
    through ``torch.ops.cuequivariance.uniform_1d``; forward and all three gradients against the CPU oracle."""
    from cuequivariance_amd import ops_torch

    ops_torch.register_ops()
    C = ops_torch.uniform_1d
    poly = channelwise_poly()
    t = U1dTables.from_polynomial(poly.flatten_coefficient_modes().squeeze_modes())
    spec = spec_from_polynomial(poly)
    g = torch.Generator().manual_seed(5)
    Z, R = 301, 17
    w = torch.randn(Z, t.width(0), dtype=torch.float64, generator=g).to(dtype)
    x1 = torch.randn(R, t.width(1), dtype=torch.float64, generator=g).to(dtype)
    x2 = torch.randn(Z, t.width(2), dtype=torch.float64, generator=g).to(dtype)
    snd = torch.randint(0, R, (Z,), generator=g, dtype=torch.int32)
    rcv = torch.sort(torch.randint(0, R, (Z,), generator=g, dtype=torch.int32))[0]
    cot = torch.randn(R, t.width(3), dtype=torch.float64, generator=g).to(dtype)
    a = [v.clone().requires_grad_(True) for v in (w, x1, x2)]
    ref = naive_segmented_polynomial(spec, a, {1: snd}, {0: R}, {0: rcv})[0]
    ref_grads = torch.autograd.grad(ref, a, cot)
    b = [v.clone().to(device).requires_grad_(True) for v in (w, x1, x2)]
    out = torch.ops.cuequivariance.uniform_1d(
        "seam", dtype, t.operand_extent, t.num_inputs, t.num_outputs, 2, list(t.buffer_dim),
        list(t.buffer_num_segments), [C.BATCH_DIM_AUTO, C.BATCH_DIM_INDEXED, C.BATCH_DIM_AUTO, C.BATCH_DIM_INDEXED],
        [-1, 0, -1, 1, R, R], list(t.dtypes), len(t.num_operands), list(t.num_operands), list(t.operations),
        list(t.num_paths), list(t.path_indices_start), list(t.path_coefficients_start), list(t.path_indices),
        list(t.path_coefficients), C.BATCH_DIM_AUTO, b + [snd.to(device), rcv.to(device)],
    )[0]
    tol = 1e-12 if dtype == torch.float64 else 1e-5
    assert out.dtype == dtype and rel_err(out, ref) <= tol
    grads = torch.autograd.grad(out, b, cot.to(device))
    for got, want in zip(grads, ref_grads):
        assert rel_err(got, want) <= tol


@pytest.mark.gpu
def test_uniform_1d_op_under_torch_compile(device):
    """The registered operator inside ``torch.compile(fullgraph=True)``: it is decomposed into the opaque launch operator;
    forward equals eager bit for bit (same kernels), and so do the gradients of this batched (atomic-free) case."""
    from cuequivariance_amd import ops_torch

    ops_torch.register_ops()
    C = ops_torch.uniform_1d
    poly = channelwise_poly()
    t = U1dTables.from_polynomial(poly.flatten_coefficient_modes().squeeze_modes())
    g = torch.Generator(device=device).manual_seed(6)
    Z = 64
    w = torch.randn(Z, t.width(0), device=device, generator=g, requires_grad=True)
    x1 = torch.randn(Z, t.width(1), device=device, generator=g, requires_grad=True)
    x2 = torch.randn(Z, t.width(2), device=device, generator=g)

    def f(w, x1, x2):
        return torch.ops.cuequivariance.uniform_1d(
            "seam", torch.float32, t.operand_extent, t.num_inputs, t.num_outputs, 0, list(t.buffer_dim),
            list(t.buffer_num_segments), [C.BATCH_DIM_AUTO] * 4, [-1] * 4, list(t.dtypes), len(t.num_operands),
            list(t.num_operands), list(t.operations), list(t.num_paths), list(t.path_indices_start),
            list(t.path_coefficients_start), list(t.path_indices), list(t.path_coefficients), C.BATCH_DIM_AUTO, [w, x1, x2])[0]

    ref = f(w, x1, x2)
    out = torch.compile(f, fullgraph=True, backend="aot_eager", dynamic=False)(w, x1, x2)
    assert torch.equal(out, ref)
    for a, b in zip(torch.autograd.grad(out.sum(), [w, x1]), torch.autograd.grad(ref.sum(), [w, x1])):
        assert torch.equal(a, b)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float64])
def test_segmented_transpose_with_frontend_info(device, dtype):
    """``segmented_transpose(x, info, True)`` with the int table of ``primitives/transpose.py:150-168``: every (u, v)
    block of the last axis is transposed (bit-exact: pure data movement), the gradient is the inverse movement."""
    from cuequivariance_amd import ops_torch

    segments = [(8, 3), (1, 5), (16, 7), (4, 1), (5, 5)]
    info, off = [], 0
    for u, v in segments:
        info.append([off, u, v, -1])
        off += u * v
    info = torch.IntTensor(info).to(device)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(37, off, generator=g, dtype=torch.float64).to(dtype)
    want = torch.cat([x[:, o:o + u * v].reshape(-1, u, v).transpose(1, 2).reshape(-1, u * v)
                      for (o, u, v, _) in info.cpu().tolist()], dim=1)
    xg = x.to(device).requires_grad_(True)
    got = ops_torch.segmented_transpose(xg, info, True)
    assert got.is_contiguous() and torch.equal(got.cpu(), want)
    (back,) = torch.autograd.grad(got, xg, got.detach())
    assert torch.equal(back.cpu(), x)
    with pytest.raises(ValueError):
        ops_torch.segmented_transpose(xg[:, :-1], info, True)


@pytest.mark.gpu
def test_fused_tensor_product_ops(device):
    """``FusedTensorProductOp3`` / ``Op4`` built from the frontend's description of a descriptor
    (``primitives/segmented_polynomial_fused_tp.py:32-48``): a linear map and a fully connected product, against the
    CPU oracle on the same descriptor."""
    from cuequivariance_amd import ops_torch

    g = torch.Generator().manual_seed(9)
    cases = (
        (cue.descriptors.linear(cue.Irreps("O3", "32x0e+32x1o"), cue.Irreps("O3", "64x0e+32x1o")),
         [1, 0, 2], "u,uv,v", ops_torch.FusedTensorProductOp3),
        (cue.descriptors.fully_connected_tensor_product(cue.Irreps("O3", "32x0e+32x1o"), cue.Irreps("O3", "0e+1o"),
                                                        cue.Irreps("O3", "32x0e+32x1o")),
         [1, 2, 0, 3], "u,v,uvw,w", ops_torch.FusedTensorProductOp4),
    )
    for e, perm, subscripts, Op in cases:
        # what the frontend passes: the irrep-component modes flattened, inputs in the order of its dispatch table
        poly = e.polynomial.flatten_coefficient_modes()
        (_, d0), = poly.operations
        d = d0.flatten_modes([m for m in d0.subscripts.modes() if m in "ijk"]).permute_operands(perm)
        assert str(d.subscripts) == subscripts
        op = Op(
            operand_segment_modes=d.subscripts.operands,
            operand_segment_offsets=[[s.start for s in ope.segment_slices()] for ope in d.operands],
            operand_segment_shapes=[ope.segments for ope in d.operands],
            path_indices=d.indices, path_coefficients=d.stacked_coefficients, math_dtype=torch.float32,
        )
        Z = 130
        ins0 = [torch.randn(1 if k == 0 else Z, ope.size, generator=g, dtype=torch.float64).float()
                for k, ope in enumerate(d0.operands[:-1])]
        ref = naive_segmented_polynomial(spec_from_polynomial(poly), ins0)[0]
        got = op(*[ins0[k].to(device) for k in perm[:-1]])
        assert got.shape == ref.shape and rel_err(got, ref) <= 1e-5


@pytest.mark.gpu
def test_triangle_entry_point(device):
    from cuequivariance_amd import ops_torch
    from oracle.triangle import triangle_multiplicative_update as oracle_trimul

    g = torch.Generator().manual_seed(4)
    D = 32
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).float().double()
    p = dict(x=r(1, 32, 32, D), p_in_weight=r(2 * D, D) / D**0.5, g_in_weight=r(2 * D, D) / D**0.5,
             p_out_weight=r(D, D) / D**0.5, g_out_weight=r(D, D) / D**0.5)
    out = ops_torch.triangle_multiplicative_update(direction="incoming", precision=ops_torch.TriMulPrecision.IEEE,
                                                   **{k: v.float().to(device) for k, v in p.items()})
    ref = oracle_trimul(direction="incoming", **p)
    assert rel_err(out, ref) <= 1e-5
