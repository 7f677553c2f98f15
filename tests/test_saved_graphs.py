"""Traced graphs that outlive the module they were traced from.

The reference's harness saves what it traced and runs the loaded copy (``torch.jit.trace`` + ``torch.jit.save`` / ``load``,
``torch.export.export`` + ``torch.export.save`` / ``load``: ``cuequivariance_torch/cuequivariance_torch/_tests/utils.py:128-210``,
modes ``jit`` and ``export``), with the original module gone by then.  Here a traced graph names its plan by text (the packed
tables of the uniform-1d path, the constructor's arguments of the dense executor), so a saved graph runs wherever
``cuequivariance_amd`` is imported: these tests load in the same process after dropping every plan, and in a child process.
"""

import gc
import importlib
import os
import subprocess
import sys

import pytest
import torch

from cuequivariance_amd import cue

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def forget_everything():
    """What a fresh process would know: no plan, no dense module."""
    gc.collect()
    u1d = importlib.import_module("cuequivariance_amd.cuet.uniform_1d")
    dense = importlib.import_module("cuequivariance_amd.cuet.dense")
    u1d._traced_plans.clear()
    u1d._plan_cache.clear()
    u1d._seam_plans.clear()
    dense._traced_modules.clear()
    gc.collect()


def channelwise(device):
    from cuequivariance_amd import cuet

    return cuet.ChannelWiseTensorProduct(cue.Irreps("O3", "32x0e+32x1o+32x2e"), cue.Irreps("O3", "0e+1o+2e"), ["0e", "1o", "2e"],
                                         layout=cue.ir_mul, shared_weights=False, internal_weights=False, device=device,
                                         dtype=torch.float32)


def channelwise_inputs(m, device, seed):
    g = torch.Generator(device=device).manual_seed(seed)
    N, Z = 40, 600
    x1 = torch.randn(N, m.irreps_in1.dim, device=device, generator=g, requires_grad=True)
    x2 = torch.randn(Z, m.irreps_in2.dim, device=device, generator=g, requires_grad=True)
    w = torch.randn(Z, m.weight_numel, device=device, generator=g, requires_grad=True)
    snd = torch.randint(0, N, (Z,), device=device, generator=g, dtype=torch.int32)
    rcv = torch.sort(torch.randint(0, N, (Z,), device=device, generator=g, dtype=torch.int32))[0]
    return x1, x2, w, snd, rcv


class Indexed(torch.nn.Module):
    def __init__(self, m, size_out):
        super().__init__()
        self.m, self.size_out = m, size_out

    def forward(self, x1, x2, w, snd, rcv):
        return self.m(x1, x2, w, indices_1=snd, indices_out=rcv, size_out=self.size_out)


def test_jit_trace_of_indexed_channelwise_survives_its_module(device, tmp_path):
    from cuequivariance_amd import _lib

    was = _lib.get_option("deterministic")
    _lib.set_option("deterministic", 1)  # (bitwise comparison of the scattered gradient)
    try:
        mod = Indexed(channelwise(device), 40)
        args = channelwise_inputs(mod.m, device, 2)
        ref = mod(*args)
        cot = torch.randn_like(ref)
        ref_grads = torch.autograd.grad(ref, args[:3], cot)
        with pytest.warns(torch.jit.TracerWarning):  # (row counts become constants of the trace, as for any shape arithmetic)
            traced = torch.jit.trace(mod, args)
        assert "u1d_launch" in str(traced.inlined_graph)
        path = str(tmp_path / "traced.ts")
        torch.jit.save(traced, path)
        del traced, mod
        forget_everything()
        loaded = torch.jit.load(path)
        out = loaded(*args)
        assert torch.equal(out, ref)
        for a, b in zip(torch.autograd.grad(out, args[:3], cot), ref_grads):
            assert torch.equal(a, b)
    finally:
        _lib.set_option("deterministic", was)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_jit_trace_of_dense_modules_and_triangle_update(device, tmp_path, dtype):
    from cuequivariance_amd import cuet

    g = torch.Generator(device=device).manual_seed(5)
    i1, i2, io = cue.Irreps("O3", "64x0e+64x1o"), cue.Irreps("O3", "0e+1o+2e"), cue.Irreps("O3", "64x0e+64x1o")

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.lin = cuet.Linear(i1, io, layout=cue.mul_ir, device=device, dtype=dtype)
            self.fc = cuet.FullyConnectedTensorProduct(i1, i2, io, layout=cue.ir_mul, device=device, dtype=dtype)
            r = lambda *shape: torch.nn.Parameter(torch.randn(*shape, device=device, generator=g).to(dtype) / 8)
            self.p_in, self.g_in, self.p_out, self.g_out = r(128, 64), r(128, 64), r(64, 64), r(64, 64)

        def forward(self, x1, x2, z):
            y = self.fc(self.lin(x1), x2)
            # (every projection given: the ones left out would be drawn at random by each call)
            t = cuet.triangle_multiplicative_update(z, direction="outgoing", p_in_weight=self.p_in, g_in_weight=self.g_in,
                                                    p_out_weight=self.p_out, g_out_weight=self.g_out)
            return y, t

    net = Net()
    x1 = torch.randn(300, i1.dim, device=device, generator=g).to(dtype).requires_grad_(True)
    x2 = torch.randn(300, i2.dim, device=device, generator=g).to(dtype).requires_grad_(True)
    z = torch.randn(1, 24, 24, 64, device=device, generator=g).to(dtype).requires_grad_(True)
    ref = net(x1, x2, z)
    cots = [torch.randn_like(r) for r in ref]
    ref_grads = torch.autograd.grad(ref, [x1, x2, z], cots)
    traced = torch.jit.trace(net, (x1, x2, z))
    text = str(traced.inlined_graph)
    assert "dense_fwd" in text and "trimul_fwd" in text
    path = str(tmp_path / "net.ts")
    torch.jit.save(traced, path)
    del traced, net
    forget_everything()
    out = torch.jit.load(path)(x1, x2, z)
    for a, b in zip(out, ref):
        assert torch.equal(a, b)
    for a, b in zip(torch.autograd.grad(out, [x1, x2, z], cots), ref_grads):
        assert torch.equal(a, b)


CHILD = r"""
import sys, torch
sys.path.insert(0, sys.argv[1])
import cuequivariance_amd.cuet  # registers the operators the saved programs call
data = torch.load(sys.argv[2] + "/inputs.pt", weights_only=True)
out = {}
ep = torch.export.load(sys.argv[2] + "/channelwise.pt2").module()
out["channelwise"] = ep(*data["channelwise"])
ep = torch.export.load(sys.argv[2] + "/dense.pt2").module()
out["dense"] = ep(*data["dense"])
ts = torch.jit.load(sys.argv[2] + "/channelwise.ts")
out["traced"] = ts(*data["channelwise"])
torch.cuda.synchronize()
torch.save(out, sys.argv[2] + "/outputs.pt")
print("child done", flush=True)
"""


def test_saved_programs_run_in_another_process(device, tmp_path):
    """``torch.export.save`` / ``torch.jit.save`` here, ``load`` and run in a child process that has never seen the modules."""
    from cuequivariance_amd import cuet

    mod = Indexed(channelwise(device), 40)
    cw_args = tuple(t.detach() for t in channelwise_inputs(mod.m, device, 9))
    g = torch.Generator(device=device).manual_seed(4)
    i1, io = cue.Irreps("O3", "64x0e+64x1o"), cue.Irreps("O3", "64x0e+64x1o")

    class Dense(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.lin = cuet.Linear(i1, io, layout=cue.mul_ir, device=device, dtype=torch.float32)
            self.fc = cuet.FullyConnectedTensorProduct(i1, cue.Irreps("O3", "0e+1o+2e"), io, layout=cue.ir_mul, device=device,
                                                       dtype=torch.float32)

        def forward(self, x1, x2):
            return self.fc(self.lin(x1), x2)

    dense = Dense()
    d_args = (torch.randn(200, i1.dim, device=device, generator=g), torch.randn(200, 9, device=device, generator=g))
    want = {"channelwise": mod(*cw_args), "dense": dense(*d_args).detach()}
    torch.export.save(torch.export.export(mod, cw_args), str(tmp_path / "channelwise.pt2"))
    torch.export.save(torch.export.export(dense, d_args), str(tmp_path / "dense.pt2"))
    with pytest.warns(torch.jit.TracerWarning):
        torch.jit.save(torch.jit.trace(mod, cw_args), str(tmp_path / "channelwise.ts"))
    torch.save({"channelwise": cw_args, "dense": d_args}, str(tmp_path / "inputs.pt"))
    script = tmp_path / "child.py"
    script.write_text(CHILD)
    print("child process: load and run the saved programs", flush=True)
    from cuequivariance_amd import jit

    env = dict(os.environ, CUEQ_AMD_JIT="1" if jit.enabled() else "0")  # (the same choice of kernels as here: results compare bit for bit)
    done = subprocess.run([sys.executable, str(script), ROOT, str(tmp_path)], capture_output=True, text=True, timeout=200, env=env)
    assert done.returncode == 0, done.stdout[-2000:] + done.stderr[-4000:]
    got = torch.load(str(tmp_path / "outputs.pt"), weights_only=True)
    assert torch.equal(got["channelwise"], want["channelwise"])
    assert torch.equal(got["traced"], want["channelwise"])
    assert torch.equal(got["dense"], want["dense"])
