"""``torch.jit.script`` of the modules, the way the reference's harness runs its ``script`` mode
(``cuequivariance_torch/_tests/utils.py:150-154``: script, ``torch.jit.save``, ``torch.jit.load``, call), for every operation the
reference tests in that mode (``tests/operations/*_test.py``: ``export_modes = ["compile", "script", "jit"]``).  The scripted
program is a stand-in that calls the eager module through one operator (``cuet/script.py``): results bit for bit those of the
eager module, first derivatives through the operator's gradient to 1e-6 of the largest value.
"""

import os

import pytest
import torch

from cuequivariance_amd import cue

pytestmark = pytest.mark.gpu


def through_script(module, tmp_path):
    scripted = torch.jit.script(module)
    name = os.path.join(tmp_path, "test.ts")
    torch.jit.save(scripted, name)
    return torch.jit.load(name)


def same(a, b, tol=1e-6):
    return (a - b).abs().max().item() <= tol * max(b.abs().max().item(), 1e-30)


def check(module, tmp_path, args, kwargs=None, params=()):
    """Eager against scripted: outputs equal, gradients of all floating-point arguments and of ``params`` (names) equal."""
    kwargs = kwargs or {}
    loaded = through_script(module, str(tmp_path))
    leaves = [a for a in list(args) + list(kwargs.values()) if isinstance(a, torch.Tensor) and a.is_floating_point()]
    for a in leaves:
        a.requires_grad_(True)
    out = module(*args, **kwargs)
    got = loaded(*args, **kwargs)
    assert got.dtype == out.dtype and torch.equal(got, out)
    cot = torch.randn_like(out)
    want = torch.autograd.grad(out, leaves + [getattr(module, n) for n in params], cot)
    have = torch.autograd.grad(got, leaves + [getattr(loaded, n) for n in params], cot)
    for h, w in zip(have, want):
        assert same(h, w)
    return loaded


def test_channelwise_and_fully_connected(device, tmp_path):
    from cuequivariance_amd import cuet

    i1, i2 = cue.Irreps("O3", "8x0e+8x1o"), cue.Irreps("O3", "0e+1o")
    g = torch.Generator(device=device).manual_seed(0)
    m = cuet.ChannelWiseTensorProduct(i1, i2, layout=cue.ir_mul, shared_weights=False, internal_weights=False, device=device)
    Z, N = 50, 7
    x1, x2 = torch.randn(N, i1.dim, device=device, generator=g), torch.randn(Z, i2.dim, device=device, generator=g)
    w = torch.randn(Z, m.weight_numel, device=device, generator=g)
    snd = torch.randint(0, N, (Z,), device=device, generator=g, dtype=torch.int32)
    rcv = torch.sort(torch.randint(0, N, (Z,), device=device, generator=g, dtype=torch.int32))[0]
    check(m, tmp_path, (x1, x2, w), dict(indices_1=snd, indices_out=rcv, size_out=N))
    shared = cuet.ChannelWiseTensorProduct(i1, i2, layout=cue.mul_ir, shared_weights=True, internal_weights=True, device=device)
    loaded = check(shared, tmp_path, (torch.randn(Z, i1.dim, device=device, generator=g), x2), params=("weight",))
    with pytest.raises(torch.jit.Error, match="Internal weights are used"):
        loaded(x1, x2, w)
    fc = cuet.FullyConnectedTensorProduct(cue.Irreps("O3", "32x0e+32x1o"), i2, cue.Irreps("O3", "32x0e+32x1o"), layout=cue.ir_mul,
                                          internal_weights=False, device=device)
    check(fc, tmp_path, (torch.randn(Z, 128, device=device, generator=g), x2, torch.randn(1, fc.weight_numel, device=device, generator=g)))


def test_linear_symmetric_contraction_and_the_small_modules(device, tmp_path):
    from cuequivariance_amd import cuet

    g = torch.Generator(device=device).manual_seed(1)
    irreps = cue.Irreps("O3", "32x0e+32x1o")
    lin = cuet.Linear(irreps, irreps, layout=cue.mul_ir, device=device)
    check(lin, tmp_path, (torch.randn(40, irreps.dim, device=device, generator=g),), params=("weight",))
    sc = cuet.SymmetricContraction(cue.Irreps("O3", "8x0e+8x1o"), cue.Irreps("O3", "8x0e"), 2, 3, layout=cue.ir_mul, device=device,
                                   dtype=torch.float32)
    idx = torch.randint(0, 3, (33,), device=device, generator=g, dtype=torch.int32)
    check(sc, tmp_path, (torch.randn(33, 32, device=device, generator=g), idx), params=("weight",))
    check(cuet.SphericalHarmonics([0, 1, 2], device=device), tmp_path, (torch.randn(21, 3, device=device, generator=g),))
    small = cue.Irreps("O3", "4x0e+4x1o+4x2e")
    check(cuet.Inversion(small, layout=cue.mul_ir, device=device), tmp_path, (torch.randn(9, small.dim, device=device, generator=g),))
    rot = cuet.Rotation(small, layout=cue.ir_mul, device=device)
    angles = torch.randn(3, 9, device=device, generator=g)
    check(rot, tmp_path, (angles[0].clone(), angles[1].clone(), angles[2].clone(), torch.randn(9, small.dim, device=device, generator=g)))
    tr = cuet.TransposeIrrepsLayout(small, source=cue.mul_ir, target=cue.ir_mul, device=device)
    check(tr, tmp_path, (torch.randn(9, small.dim, device=device, generator=g),))
    same_layout = cuet.TransposeIrrepsLayout(small, source=cue.ir_mul, target=cue.ir_mul, device=device)
    check(same_layout, tmp_path, (torch.randn(9, small.dim, device=device, generator=g),))


def test_a_scripted_program_whose_module_is_gone_says_so(device, tmp_path):
    from cuequivariance_amd import cuet
    from cuequivariance_amd.cuet import script

    m = cuet.SphericalHarmonics([1], device=device)
    loaded = through_script(m, str(tmp_path))
    v = torch.randn(4, 3, device=device)
    assert torch.equal(loaded(v), m(v))
    script._live.pop(m._script_key)
    with pytest.raises(RuntimeError, match="not alive in this process"):
        loaded(v)


def test_segmented_polynomial_with_lists_and_dictionaries(device, tmp_path):
    """``cuet.SegmentedPolynomial`` scripted, called the way the reference's primitive tests call it
    (``tests/primitives/segmented_polynomial_test.py:284``): a list of inputs, dictionaries of index tensors and output shapes."""
    from cuequivariance_amd import cuet

    e = cue.descriptors.channelwise_tensor_product(cue.Irreps("O3", "8x0e+8x1o"), cue.Irreps("O3", "0e+1o"))
    m = cuet.SegmentedPolynomial(e.polynomial, method="uniform_1d", math_dtype=torch.float32)
    loaded = through_script(m, str(tmp_path))
    g = torch.Generator(device=device).manual_seed(2)
    Z, N = 60, 9
    ins = [torch.randn(Z, e.inputs[0].dim, device=device, generator=g, requires_grad=True),
           torch.randn(N, e.inputs[1].dim, device=device, generator=g, requires_grad=True),
           torch.randn(Z, e.inputs[2].dim, device=device, generator=g, requires_grad=True)]
    snd = torch.randint(0, N, (Z,), device=device, generator=g, dtype=torch.int32)
    rcv = torch.randint(0, N, (Z,), device=device, generator=g, dtype=torch.int64)
    shape = torch.empty(N, 1, device=device)
    want = m(ins, {1: snd}, {0: shape}, {0: rcv})
    got = loaded(ins, {1: snd}, {0: shape}, {0: rcv})
    assert len(got) == 1 and torch.equal(got[0], want[0])
    cot = torch.randn_like(want[0])
    for h, w in zip(torch.autograd.grad(got[0], ins, cot), torch.autograd.grad(want[0], ins, cot)):
        assert same(h, w)
    plain = loaded([ins[0], ins[1][:1].expand(Z, -1).contiguous(), ins[2]])
    assert torch.equal(plain[0], m([ins[0], ins[1][:1].expand(Z, -1).contiguous(), ins[2]])[0])
