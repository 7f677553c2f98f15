"""Layers built on the tensor-product modules.

Mirror of ``cuequivariance_torch/cuequivariance_torch/layers/batchnorm.py:26-226`` (``BatchNorm``) and
``layers/tp_conv_fully_connected.py:29-276`` (``FullyConnectedTensorProductConv``): same constructor arguments,
buffers / parameters (``running_mean``, ``running_var``, ``weight``, ``bias``, ``mlp``) and forward signatures.

* ``BatchNorm`` is element-wise torch arithmetic in the reference too; here the per-irrep loops are replaced by three
  small constant maps (element -> channel, channel -> scalar slot, the component-averaging matrix), so a forward is a
  handful of tensor operations whatever the number of irreps.
* ``FullyConnectedTensorProductConv`` hands the gather of source rows and the reduction onto destination rows to the
  uniform-1d kernels (an indexed input and an indexed output of the fully connected product with per-edge weights):
  neither the ``(edges, in_irreps.dim)`` nor the ``(edges, out_irreps.dim)`` intermediate of the reference exists.
"""

from __future__ import annotations

from typing import Optional, Sequence, Union

import torch
from torch import nn

from .. import cue
from .operations import FullyConnectedTensorProduct, _assert_same_group, _default_irreps, _default_layout

__all__ = ["BatchNorm", "FullyConnectedTensorProductConv"]


class BatchNorm(nn.Module):
    """Batch normalisation of a tensor of irreps: scalar channels are centred, every channel (one per irrep copy) is
    divided by the root of its mean squared component, then scaled (``weight``, one per channel) and, for scalars,
    shifted (``bias``).  ``instance=True`` takes the statistics per batch element; ``reduce`` says how the squared norm
    is reduced over the sample axis ("mean" or "max")."""

    def __init__(self, irreps: cue.Irreps, *, layout: cue.IrrepsLayout = None, eps: float = 1e-5, momentum: float = 0.1,
                 affine: bool = True, reduce: str = "mean", instance: bool = False, include_bias: bool = True):
        super().__init__()
        self.layout = _default_layout(layout)
        (self.irreps,) = _default_irreps(irreps)
        self.eps, self.momentum, self.affine, self.instance, self.include_bias = eps, momentum, affine, instance, include_bias
        assert isinstance(reduce, str), "reduce should be passed as a string value"
        assert reduce in ["mean", "max"], "reduce needs to be 'mean' or 'max'"
        self.reduce = reduce

        channel_of, scalar_slot, dims = [], [], []
        nch = nsc = 0
        for mul, ir in self.irreps:
            d = ir.dim
            u = torch.arange(mul)
            block = u.repeat_interleave(d) if self.layout == cue.mul_ir else u.repeat(d)  # (u, i) or (i, u) order
            channel_of.append(nch + block)
            scalar_slot += list(range(nsc, nsc + mul)) if ir.is_scalar() else [-1] * mul
            dims += [d] * mul
            nch += mul
            nsc += mul if ir.is_scalar() else 0
        channel_of = torch.cat(channel_of) if channel_of else torch.zeros(0, dtype=torch.long)
        scalar_slot = torch.tensor(scalar_slot, dtype=torch.long)
        self.num_features, self.num_scalar = nch, nsc
        self.register_buffer("_channel_of", channel_of, persistent=False)  # element -> channel
        self.register_buffer("_scalar_channels", torch.nonzero(scalar_slot >= 0).flatten(), persistent=False)
        averaging = torch.zeros(channel_of.numel(), nch, dtype=torch.float64)  # (rounded to the input type at use)
        averaging[torch.arange(channel_of.numel()), channel_of] = 1.0 / torch.tensor(dims, dtype=torch.float64)[channel_of]
        self.register_buffer("_averaging", averaging, persistent=False)  # (dim, channels): mean over the components

        if self.instance:
            self.register_buffer("running_mean", None)
            self.register_buffer("running_var", None)
        else:
            self.register_buffer("running_mean", torch.zeros(nsc))
            self.register_buffer("running_var", torch.ones(nch))
        if affine:
            self.weight = nn.Parameter(torch.ones(nch))
            if include_bias:
                self.bias = nn.Parameter(torch.zeros(nsc))
        else:
            self.register_parameter("weight", None)
            if include_bias:
                self.register_parameter("bias", None)

    def extra_repr(self) -> str:
        return f"{self.irreps}, layout={self.layout}, eps={self.eps}, momentum={self.momentum}"

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        shape = input.shape
        batch, dim = shape[0], shape[-1]
        torch._assert(dim == self._channel_of.numel(), f"the last dimension must be {self._channel_of.numel()}, got {dim}")
        x = input.reshape(batch, -1, dim)  # [batch, sample, elements]
        stats = self.training or self.instance
        nch, sc = self.num_features, self._scalar_channels
        avg = self._averaging.to(x.dtype)

        # centre the scalar channels
        if self.num_scalar > 0:
            if stats:
                per_channel = x @ avg  # scalars have one component: their value
                mean = per_channel[..., sc].mean(1) if self.instance else per_channel[..., sc].mean((0, 1))  # [(batch,) scalars]
                if not self.instance and self.training:
                    self.running_mean.copy_((1 - self.momentum) * self.running_mean + self.momentum * mean.detach())
            else:
                mean = self.running_mean
            full = x.new_zeros(mean.shape[:-1] + (nch,))
            full[..., sc] = mean.to(x.dtype)
            shift = full[..., self._channel_of]  # [(batch,) elements]
            x = x - (shift.unsqueeze(1) if self.instance else shift)

        # mean squared component per channel
        if stats:
            norm = (x * x) @ avg  # [batch, sample, channels]
            norm = norm.mean(1) if self.reduce == "mean" else norm.max(1).values  # [batch, channels]
            if not self.instance:
                norm = norm.mean(0)
                if self.training:
                    self.running_var.copy_((1 - self.momentum) * self.running_var + self.momentum * norm.detach())
        else:
            norm = self.running_var
        scale = (norm + self.eps).pow(-0.5)  # [(batch,) channels]
        if self.affine:
            scale = scale * self.weight
        scale = scale.to(x.dtype)[..., self._channel_of]
        x = x * (scale.unsqueeze(1) if self.instance else scale)

        if self.affine and self.include_bias and self.num_scalar > 0:
            full = x.new_zeros(nch)
            full[sc] = self.bias.to(x.dtype)
            x = x + full[self._channel_of]
        return x.reshape(shape)


class FullyConnectedTensorProductConv(nn.Module):
    """Message passing with a fully connected tensor product (DiffDock-style): for every destination node the sum (or
    mean) over its edges of ``h_src (x) Y(edge)`` with per-edge path weights, which are either given (``mlp_channels=None``:
    ``edge_emb`` has ``tp.weight_numel`` columns) or produced by an MLP from the edge embedding and optional scalar
    features of the two end points.  ``graph = ((src, dst), (num_src_nodes, num_dst_nodes))``."""

    def __init__(self, in_irreps: cue.Irreps, sh_irreps: cue.Irreps, out_irreps: cue.Irreps, batch_norm: bool = True,
                 mlp_channels: Optional[Sequence[int]] = None,
                 mlp_activation: Union[nn.Module, Sequence[nn.Module], None] = nn.GELU(),
                 layout: cue.IrrepsLayout = None, use_fallback: Optional[bool] = None):
        super().__init__()
        in_irreps, out_irreps, sh_irreps = _default_irreps(in_irreps, out_irreps, sh_irreps)
        _assert_same_group(in_irreps, out_irreps, sh_irreps)
        self.in_irreps, self.out_irreps, self.sh_irreps = in_irreps, out_irreps, sh_irreps
        self.layout = _default_layout(layout)
        self.tp = FullyConnectedTensorProduct(in_irreps, sh_irreps, out_irreps, layout=self.layout, shared_weights=False,
                                              use_fallback=use_fallback)
        self.batch_norm = BatchNorm(out_irreps, layout=self.layout) if batch_norm else None

        if mlp_activation is None:
            activations = []
        elif hasattr(mlp_activation, "__len__") and hasattr(mlp_activation, "__getitem__"):
            activations = list(mlp_activation)
        else:
            activations = [mlp_activation]
        if mlp_channels is not None:
            widths = list(mlp_channels) + [self.tp.weight_numel]
            stages = []
            for i in range(len(widths) - 1):
                stages.append(nn.Linear(widths[i], widths[i + 1]))
                if i != len(widths) - 2:
                    stages.extend(activations)
            self.mlp = nn.Sequential(*stages)
        else:
            self.mlp = None

    def _path_weights(self, edge_emb, src, dst, src_scalars, dst_scalars):
        if self.mlp is None:
            return edge_emb
        if src_scalars is None and dst_scalars is None:
            return self.mlp(edge_emb)
        # first layer applied per component before indexing (smaller GEMMs): weight columns are edge | source | destination
        first = self.mlp[0]
        sizes = (edge_emb.size(-1), 0 if src_scalars is None else src_scalars.size(-1),
                 0 if dst_scalars is None else dst_scalars.size(-1))
        w_edge, w_src, w_dst = torch.split(first.weight, sizes, dim=-1)
        hidden = edge_emb @ w_edge.T + first.bias
        if src_scalars is not None:
            hidden = hidden + (src_scalars @ w_src.T)[src]
        if dst_scalars is not None:
            hidden = hidden + (dst_scalars @ w_dst.T)[dst]
        return self.mlp[1:](hidden)

    def forward(self, src_features: torch.Tensor, edge_sh: torch.Tensor, edge_emb: torch.Tensor,
                graph: tuple, src_scalars: Optional[torch.Tensor] = None, dst_scalars: Optional[torch.Tensor] = None,
                reduce: str = "mean", edge_envelope: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Arguments as in the reference (``layers/tp_conv_fully_connected.py:156-276``).  Destination ids outside
        ``[0, num_dst_nodes)`` raise an error in eager mode; while the current stream is being captured into a HIP graph the
        grouping of the edges by destination is recorded as device work that cannot report them: such edges are left out of
        every destination row, at capture and at every replay."""
        edge_width = edge_emb.size(-1)
        if self.mlp is None:
            if self.tp.weight_numel != edge_width:
                raise RuntimeError(
                    f"When MLP is not present, edge_emb's last dimension must equal tp.weight_numel (but got {edge_width} "
                    f"and {self.tp.weight_numel})")
        else:
            total = edge_width + (0 if src_scalars is None else src_scalars.size(-1)) + (0 if dst_scalars is None else dst_scalars.size(-1))
            if self.mlp[0].in_features != total:
                raise RuntimeError(
                    f"The size of MLP's input layer ({self.mlp[0].in_features}) does not match the total number of scalar "
                    f"features from edge_emb, src_scalars and dst_scalars ({total})")
        if reduce not in ["mean", "sum"]:
            raise RuntimeError(f"reduce argument must be either 'mean' or 'sum', got {reduce}.")
        (src, dst), (num_src_nodes, num_dst_nodes) = graph

        weights = self._path_weights(edge_emb, src, dst, src_scalars, dst_scalars)
        if edge_envelope is not None:  # the product is linear in the harmonics: fold the per-edge factor in there
            edge_sh = edge_sh * edge_envelope.view(-1, 1)
        out = self.tp(src_features, edge_sh, weights, indices_1=src, indices_out=dst, size_out=num_dst_nodes)
        if reduce == "mean":
            degree = torch.bincount(dst.long(), minlength=num_dst_nodes).clamp(min=1)
            out = out / degree.to(out.dtype).unsqueeze(1)
        if self.batch_norm is not None:
            out = self.batch_norm(out)
        return out
