"""``cuet.layers``: BatchNorm against library routines and closed forms (CPU), the convolution layer against the CPU
oracle of the tensor product with explicit gather / scatter (GPU).  Reference behaviour:
``cuequivariance_torch/layers/batchnorm.py:26-226``, ``layers/tp_conv_fully_connected.py:29-276``."""

import copy

import pytest
import torch
import torch.nn.functional as F

from cuequivariance_amd import cue, cuet
from oracle.naive import naive_segmented_polynomial, spec_from_polynomial


@pytest.mark.parametrize("layout", [cue.mul_ir, cue.ir_mul])
def test_batchnorm_scalars_are_library_batch_norm_and_vectors_closed_form(layout):
    torch.manual_seed(0)
    bn = cuet.layers.BatchNorm(cue.Irreps("O3", "5x0e+3x1o+2x0e"), layout=layout)
    with torch.no_grad():
        bn.weight.copy_(torch.rand(10) + 0.5)
        bn.bias.copy_(torch.randn(7))
    x = torch.randn(40, 5 + 9 + 2, dtype=torch.float64)
    bn = bn.double()
    y = bn(x)
    # the seven scalar channels (5x0e and 2x0o): torch's batch_norm in training mode (biased variance) is the same map
    sc = torch.cat([x[:, :5], x[:, 14:]], dim=1)
    want = F.batch_norm(sc, None, None, torch.cat([bn.weight[:5], bn.weight[8:]]), bn.bias, True, 0.1, bn.eps)
    torch.testing.assert_close(torch.cat([y[:, :5], y[:, 14:]], dim=1), want, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(bn.running_mean, 0.1 * sc.mean(0), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(torch.cat([bn.running_var[:5], bn.running_var[8:]]), 0.9 + 0.1 * sc.var(0, unbiased=False),
                               rtol=1e-12, atol=1e-12)
    # vector channels: not centred, divided by the root mean square over batch and components
    v = x[:, 5:14].reshape(40, 3, 3) if layout == cue.mul_ir else x[:, 5:14].reshape(40, 3, 3).transpose(1, 2)  # [z, u, i]
    scale = (v.pow(2).mean((0, 2)) + bn.eps).rsqrt() * bn.weight[5:8]
    got = y[:, 5:14].reshape(40, 3, 3) if layout == cue.mul_ir else y[:, 5:14].reshape(40, 3, 3).transpose(1, 2)
    torch.testing.assert_close(got, v * scale.view(1, 3, 1), rtol=1e-12, atol=1e-12)
    # rotating the vectors (any orthogonal matrix on the component axis) commutes with the layer
    q, _ = torch.linalg.qr(torch.randn(3, 3, dtype=torch.float64))
    xr = x.clone()
    vr = torch.einsum("zui,ij->zuj", v, q)
    xr[:, 5:14] = (vr if layout == cue.mul_ir else vr.transpose(1, 2)).reshape(40, 9)
    bn2 = copy.deepcopy(bn)
    yr = bn2(xr)
    gr = yr[:, 5:14].reshape(40, 3, 3) if layout == cue.mul_ir else yr[:, 5:14].reshape(40, 3, 3).transpose(1, 2)
    torch.testing.assert_close(gr, torch.einsum("zui,ij->zuj", got, q), rtol=1e-10, atol=1e-10)
    # evaluation mode uses the running statistics
    bn.eval()
    ye = bn(x)
    want = F.batch_norm(sc, bn.running_mean, torch.cat([bn.running_var[:5], bn.running_var[8:]]),
                        torch.cat([bn.weight[:5], bn.weight[8:]]), bn.bias, False, 0.1, bn.eps)
    torch.testing.assert_close(torch.cat([ye[:, :5], ye[:, 14:]], dim=1), want, rtol=1e-12, atol=1e-12)


def test_batchnorm_instance_and_max_reduce():
    torch.manual_seed(1)
    x = torch.randn(6, 11, 4 + 6, dtype=torch.float64)  # [batch, sample, 4x0e+2x1o]
    inst = cuet.layers.BatchNorm(cue.Irreps("O3", "4x0e+2x1o"), layout=cue.mul_ir, instance=True, affine=False).double()
    y = inst(x)
    want = F.instance_norm(x[..., :4].transpose(1, 2), eps=inst.eps).transpose(1, 2)  # statistics over the sample axis
    torch.testing.assert_close(y[..., :4], want, rtol=1e-12, atol=1e-12)
    assert inst.running_mean is None and inst.weight is None
    mx = cuet.layers.BatchNorm(cue.Irreps("O3", "4x0e+2x1o"), layout=cue.mul_ir, reduce="max", affine=False).double()
    y = mx(x)
    v = x[..., 4:].reshape(6, 11, 2, 3)
    norm = v.pow(2).mean(3).max(1).values.mean(0)  # component mean, max over samples, mean over the batch
    torch.testing.assert_close(y[..., 4:].reshape(6, 11, 2, 3), v * (norm + mx.eps).rsqrt().view(1, 1, 2, 1), rtol=1e-12, atol=1e-12)
    with pytest.raises(AssertionError):
        cuet.layers.BatchNorm(cue.Irreps("O3", "1x0e"), layout=cue.mul_ir, reduce="sum")


@pytest.mark.gpu
@pytest.mark.parametrize("layout", [cue.ir_mul, cue.mul_ir])
@pytest.mark.parametrize("mode", ["weights", "mlp", "mlp_split"])
def test_tensor_product_conv_against_oracle(device, layout, mode):
    """out[d] = reduce over edges (s -> d) of TP(h[s], sh[e]; w[e]), then batch norm: the tensor product from the CPU
    oracle on explicitly gathered rows, the reduction with ``index_add_``, the MLP and batch norm as plain torch."""
    g = torch.Generator().manual_seed(31)
    i_in, i_sh, i_out = cue.Irreps("O3", "6x0e+4x1o"), cue.Irreps("O3", "0e+1o"), cue.Irreps("O3", "6x0e+4x1o")
    ns, nd, E = 23, 17, 140
    mlp = None if mode == "weights" else [5 + (7 if mode == "mlp_split" else 0), 12]
    conv = cuet.layers.FullyConnectedTensorProductConv(i_in, i_sh, i_out, mlp_channels=mlp, mlp_activation=torch.nn.SiLU(),
                                                       layout=layout)
    ref_conv = copy.deepcopy(conv)
    conv = conv.to(device)
    h = torch.randn(ns, i_in.dim, generator=g)
    sh = torch.randn(E, i_sh.dim, generator=g)
    src, dst = torch.randint(0, ns, (E,), generator=g), torch.randint(0, nd - 2, (E,), generator=g)  # two nodes without edges
    env = torch.rand(E, generator=g)
    emb = torch.randn(E, conv.tp.weight_numel if mlp is None else 5, generator=g)
    ss, ds = (torch.randn(ns, 3, generator=g), torch.randn(nd, 4, generator=g)) if mode == "mlp_split" else (None, None)

    # reference evaluation
    if mlp is None:
        w = emb
    elif mode == "mlp":
        w = ref_conv.mlp(emb)
    else:
        w = ref_conv.mlp(torch.hstack((emb, ss[src], ds[dst])))  # the documented equivalent of the split first layer
    e = cue.descriptors.fully_connected_tensor_product(i_in, i_sh, i_out)
    to_ir_mul = (lambda t, irreps: t) if layout == cue.ir_mul else (
        lambda t, irreps: torch.cat([t[:, o:o + m * ir.dim].reshape(-1, m, ir.dim).transpose(1, 2).reshape(-1, m * ir.dim)
                                     for o, (m, ir) in zip(_offsets(irreps), irreps)], dim=1))
    from_ir_mul = (lambda t, irreps: t) if layout == cue.ir_mul else (
        lambda t, irreps: torch.cat([t[:, o:o + m * ir.dim].reshape(-1, ir.dim, m).transpose(1, 2).reshape(-1, m * ir.dim)
                                     for o, (m, ir) in zip(_offsets(irreps), irreps)], dim=1))
    msg = naive_segmented_polynomial(spec_from_polynomial(e.polynomial),
                                     [w.double(), to_ir_mul(h, i_in)[src].double(), to_ir_mul(sh, i_sh).double()])[0]
    msg = from_ir_mul(msg, i_out) * env.double().view(-1, 1)
    summed = torch.zeros(nd, i_out.dim, dtype=torch.float64).index_add_(0, dst, msg)
    mean = summed / torch.bincount(dst, minlength=nd).clamp(min=1).double().view(-1, 1)
    want = ref_conv.batch_norm.double()(mean)

    dev = lambda t: None if t is None else t.to(device)
    got = conv(dev(h), dev(sh), dev(emb), ((dev(src), dev(dst)), (ns, nd)), dev(ss), dev(ds), reduce="mean", edge_envelope=dev(env))
    assert got.shape == (nd, i_out.dim)
    err = (got.detach().cpu().double() - want).abs().max().item() / want.abs().max().item()
    assert err <= 1e-5, err
    # gradients reach the MLP (or the given weights) and the node features
    params = [p for p in conv.parameters() if p.requires_grad]
    hg = dev(h).requires_grad_(True)
    out = conv(hg, dev(sh), dev(emb), ((dev(src), dev(dst)), (ns, nd)), dev(ss), dev(ds), reduce="sum")
    grads = torch.autograd.grad(out.square().sum(), [hg] + params, allow_unused=True)
    assert grads[0] is not None and torch.isfinite(grads[0]).all()
    with pytest.raises(RuntimeError):
        conv(dev(h), dev(sh), dev(emb), ((dev(src), dev(dst)), (ns, nd)), reduce="prod")


def _offsets(irreps):
    out, o = [], 0
    for m, ir in irreps:
        out.append(o)
        o += m * ir.dim
    return out
