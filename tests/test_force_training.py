"""One interaction layer in the style of MACE, end to end under force training: positions -> spherical harmonics ->
indexed channel-wise product with per-edge weights -> Linear -> symmetric contraction -> element-dependent skip
connection (fully connected product with node attributes) -> energy; forces = -dE/dpositions with ``create_graph=True``;
gradient of a loss on energy and forces with respect to every weight.  The same pipeline through the CPU oracle in
float64 is the reference: every module has to compose under a second backward."""

import pytest
import torch

from cuequivariance_amd import cue
from oracle.naive import naive_segmented_polynomial, spec_from_polynomial

pytestmark = pytest.mark.gpu


def test_mace_style_layer_energy_and_force_gradients(device):
    from cuequivariance_amd import cuet

    dt = torch.float64
    mul, nel = 16, 3
    feats = cue.Irreps("O3", f"{mul}x0e+{mul}x1o")
    sh_irreps = cue.Irreps("O3", "0e+1o+2e")
    sh = cuet.SphericalHarmonics([0, 1, 2], normalize=True, device=device)
    tp = cuet.ChannelWiseTensorProduct(feats, sh_irreps, "0e+1o", layout=cue.ir_mul, shared_weights=False, internal_weights=False,
                                       device=device, dtype=dt)
    lin = cuet.Linear(tp.irreps_out, feats, layout=cue.ir_mul, internal_weights=False, method="fused_tp")
    sc = cuet.SymmetricContraction(feats, cue.Irreps("O3", f"{mul}x0e"), 2, nel, layout_in=cue.ir_mul, layout_out=cue.ir_mul,
                                   dtype=dt, device=device)
    skip = cuet.FullyConnectedTensorProduct(feats, cue.Irreps("O3", f"{nel}x0e"), cue.Irreps("O3", f"{mul}x0e"), layout=cue.ir_mul,
                                            internal_weights=False)
    g = torch.Generator().manual_seed(21)
    N, E = 12, 60
    pos = torch.randn(N, 3, generator=g, dtype=dt)
    snd = torch.randint(0, N, (E,), generator=g)
    rcv = torch.sort(torch.randint(0, N, (E,), generator=g))[0]
    keep = snd != rcv
    snd, rcv = snd[keep], rcv[keep]
    E = int(snd.numel())
    species = torch.randint(0, nel, (N,), generator=g)
    attrs = torch.nn.functional.one_hot(species, nel).to(dt)
    h = torch.randn(N, feats.dim, generator=g, dtype=dt)
    radial = torch.randn(3, tp.weight_numel, generator=g, dtype=dt) * 0.3   # per-edge weights = radial basis @ this
    w_lin = torch.randn(1, lin.weight_numel, generator=g, dtype=dt)
    w_sc = sc.weight.detach().cpu().clone()
    w_skip = torch.randn(1, skip.weight_numel, generator=g, dtype=dt)
    f_target = torch.randn(N, 3, generator=g, dtype=dt)

    specs = {"sh": spec_from_polynomial(sh.f._polynomial_orig), "tp": spec_from_polynomial(tp.f._polynomial_orig),
             "lin": spec_from_polynomial(lin.f._polynomial_orig), "sc": spec_from_polynomial(sc.f._polynomial_orig),
             "skip": spec_from_polynomial(skip.f_per_sample._polynomial)}

    def pipeline(ops, pos_, params, dev_):
        radial_, w_lin_, w_sc_, w_skip_ = params
        vec = pos_[rcv.to(dev_)] - pos_[snd.to(dev_)]
        r = vec.norm(dim=1, keepdim=True)
        y = ops["sh"](vec)
        basis = torch.cat([torch.exp(-r), torch.exp(-2 * r), r * torch.exp(-r)], 1)
        m = ops["tp"](h.to(dev_), y, basis @ radial_)
        a = ops["lin"](m, w_lin_)
        b = ops["sc"](a, w_sc_)
        e_node = (b + ops["skip"](a, attrs.to(dev_), w_skip_)).sum(1)
        return e_node.sum()

    def loss_grads(ops, dev_):
        p = pos.clone().to(dev_).requires_grad_(True)
        params = [t.clone().to(dev_).requires_grad_(True) for t in (radial, w_lin, w_sc, w_skip)]
        energy = pipeline(ops, p, params, dev_)
        (de,) = torch.autograd.grad(energy, [p], create_graph=True)
        loss = energy * 0.1 + ((-de - f_target.to(dev_)) ** 2).sum()
        return [energy.detach(), -de.detach()] + list(torch.autograd.grad(loss, params))

    cpu = torch.device("cpu")
    oracle_ops = {
        "sh": lambda v: naive_segmented_polynomial(specs["sh"], [v / v.norm(dim=1, keepdim=True)])[0],  # (normalize=True)
        "tp": lambda x1, x2, w: naive_segmented_polynomial(specs["tp"], [w, x1, x2], {1: snd}, {0: N}, {0: rcv})[0],
        "lin": lambda x, w: naive_segmented_polynomial(specs["lin"], [w, x])[0],
        "sc": lambda x, w: naive_segmented_polynomial(specs["sc"], [w.reshape(nel, -1), x], {0: species}, {}, {})[0],
        "skip": lambda x1, x2, w: naive_segmented_polynomial(specs["skip"], [w, x1, x2])[0],
    }
    snd_d, rcv_d, species_d = snd.to(device).int(), rcv.to(device).int(), species.to(device).int()

    def sc_gpu(x, w):
        return torch.func.functional_call(sc, {"weight": w}, (x, species_d))

    gpu_ops = {
        "sh": lambda v: sh(v),
        "tp": lambda x1, x2, w: tp(x1, x2, w, indices_1=snd_d, indices_out=rcv_d, size_out=N),
        "lin": lambda x, w: lin(x, w),
        "sc": sc_gpu,
        "skip": lambda x1, x2, w: skip(x1, x2, w),
    }
    want = loss_grads(oracle_ops, cpu)
    got = loss_grads(gpu_ops, device)
    names = ("energy", "forces", "d/d radial", "d/d linear weights", "d/d contraction weights", "d/d skip weights")
    for name, p, q in zip(names, got, want):
        err = (p.cpu() - q).abs().max().item() / max(q.abs().max().item(), 1e-30)
        assert err <= 1e-10, (name, err)
