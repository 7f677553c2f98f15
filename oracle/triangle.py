"""CPU oracle of the triangle multiplicative update (test infrastructure only - the product never imports this).

Plain torch restatement of the reference's open algorithm
(``cuequivariance_jax/cuequivariance_jax/triangle/_triangle_multiplicative_update.py:371-417``) from its stage
references: LayerNorm with biased variance ``_layer_norm_transpose.py:196-209``, gated dual projection
``_sigmoid_gated_dual_gemm.py:127-150`` (mask multiplies the gated product), contraction ``:393-397``, and the
output gate that reads the *normalised* input ``:408-417``.  Evaluated in the dtype of the inputs given (use float64
inputs rounded to the tested dtype); gradients by torch autograd of the same formula.
"""

from __future__ import annotations

import torch


def layer_norm(x, w, b, eps):
    mean = x.mean(dim=-1, keepdim=True)
    xc = x - mean
    var = (xc * xc).mean(dim=-1, keepdim=True)
    y = xc / torch.sqrt(var + eps)
    if w is not None:
        y = y * w
    if b is not None:
        y = y + b
    return y


def triangle_multiplicative_update(x, direction="outgoing", mask=None, norm_in_weight=None, norm_in_bias=None,
                                   p_in_weight=None, p_in_bias=None, g_in_weight=None, g_in_bias=None,
                                   norm_out_weight=None, norm_out_bias=None, p_out_weight=None, p_out_bias=None,
                                   g_out_weight=None, g_out_bias=None, eps=1e-5):
    """x (B, N, N, D); projection weights are required (the reference draws them at random when absent)."""
    xh = layer_norm(x, norm_in_weight, norm_in_bias, eps)
    gate = xh @ g_in_weight.T
    proj = xh @ p_in_weight.T
    if g_in_bias is not None:
        gate = gate + g_in_bias
    if p_in_bias is not None:
        proj = proj + p_in_bias
    ab = torch.sigmoid(gate) * proj
    if mask is not None:
        ab = ab * mask[..., None]
    D = x.shape[-1]
    a, b = ab[..., :D], ab[..., D:]
    if direction == "outgoing":
        t = torch.einsum("bikd,bjkd->bijd", a, b)
    elif direction == "incoming":
        t = torch.einsum("bkid,bkjd->bijd", a, b)
    else:
        raise ValueError(direction)
    y = layer_norm(t, norm_out_weight, norm_out_bias, eps)
    gate = xh @ g_out_weight.T
    proj = y @ p_out_weight.T
    if g_out_bias is not None:
        gate = gate + g_out_bias
    if p_out_bias is not None:
        proj = proj + p_out_bias
    return torch.sigmoid(gate) * proj
