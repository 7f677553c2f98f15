"""Triangle multiplicative update (pair-representation update of AlphaFold-style models) on HIP kernels.

``triangle_multiplicative_update`` keeps the signature, defaults and error behaviour of
``cuequivariance_torch/cuequivariance_torch/primitives/triangle.py:138-262``; the computation is the one the
reference states in the open
``cuequivariance_jax/cuequivariance_jax/triangle/_triangle_multiplicative_update.py:371-417``::

    xh  = LayerNorm(x; norm_in)                                            (B, N, N, D)
    ab  = sigmoid(xh G_in^T + b) * (xh P_in^T + b) * mask, stored (2D, B, N, N);  a, b = split(ab)
    t   = einsum("dbik,dbjk->dbij", a, b)   (outgoing)   /  einsum("dbki,dbkj->dbij", a, b)   (incoming)
    y   = LayerNorm over d of t, stored (B, N, N, D)
    out = sigmoid(xh G_out^T + b) * (y P_out^T + b)       -- the output gate reads the normalised input xh

Every stage is a HIP kernel reached through the C ABI (``cueq_gemm_nt``, ``cueq_layer_norm_*``, ``cueq_gate_*``,
``cueq_transpose``, ``cueq_sum_*``); torch only owns the buffers.  Inputs float32 or bfloat16, fp32 accumulation;
intermediate tensors are kept in the input dtype like the reference does; the projection accumulators stay in registers
(``cueq_dual_gate`` fuses both projections with the gate and recomputes them in the backward).
"""

from __future__ import annotations

import enum
import math
from typing import List, Optional

import torch

from .. import _lib

__all__ = ["triangle_multiplicative_update", "TriMulPrecision"]


class TriMulPrecision(enum.IntEnum):
    """Matrix-multiplication precision request (reference ``primitives/triangle.py:24-31``).  The MFMA kernels
    here compute float32 inputs in IEEE float32 and bfloat16 inputs with float32 accumulation whatever is asked."""

    NONE = -1
    DEFAULT = 0
    TF32 = 1
    TF32x3 = 2
    IEEE = 3


_CODE = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16, torch.float16: _lib.F16}
_TWO_BYTE = (torch.bfloat16, torch.float16)  # the matrix-core kernels for 2-byte elements take either format


def _stream(t: torch.Tensor):
    return torch.cuda.current_stream(t.device).cuda_stream


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


# ---------------------------------------------------------------------------------------------
# thin wrappers over the C ABI (shapes checked here, before any launch)
# ---------------------------------------------------------------------------------------------
def gemm_nt(A: torch.Tensor, B: torch.Tensor, out_dtype: torch.dtype, out: Optional[torch.Tensor] = None,
            accumulate: bool = False, alpha: float = 1.0, trans_a: bool = False, trans_b: bool = False) -> torch.Tensor:
    """``C[b] = alpha * A[b] @ B[b]^T (+ C[b])`` for ``A (batch, M, K)``, ``B (batch, N, K)`` (or 2-D, batch 1);
    ``trans_a`` / ``trans_b``: that operand is given as ``(batch, K, M)`` / ``(batch, K, N)`` instead."""
    squeeze = A.dim() == 2
    if squeeze:
        A, B = A.unsqueeze(0), B.unsqueeze(0)
    assert A.dim() == 3 and B.dim() == 3 and A.shape[0] == B.shape[0], (A.shape, B.shape)
    assert A.dtype == B.dtype and A.stride(2) == 1 and B.stride(2) == 1
    batch = A.shape[0]
    K, M = (A.shape[1], A.shape[2]) if trans_a else (A.shape[2], A.shape[1])
    Kb, N = (B.shape[1], B.shape[2]) if trans_b else (B.shape[2], B.shape[1])
    assert K == Kb, (A.shape, B.shape, trans_a, trans_b)
    if out is None:
        assert not accumulate
        out = torch.empty(batch, M, N, dtype=out_dtype, device=A.device)
    else:
        out = out.view(batch, M, N)
        assert out.dtype == out_dtype and out.is_contiguous()
    _lib.check(
        _lib.load().cueq_gemm(
            _CODE[A.dtype], _CODE[out_dtype], int(trans_a), int(trans_b), M, N, K, A.data_ptr(), A.stride(1),
            A.stride(0) if batch > 1 else 0, B.data_ptr(), B.stride(1), B.stride(0) if batch > 1 else 0, out.data_ptr(), N, M * N,
            batch, float(alpha), int(accumulate), _stream(A),
        ),
        "cueq_gemm",
    )
    return out[0] if squeeze else out


def transpose(x: torch.Tensor) -> torch.Tensor:
    """Swap the last two axes of a contiguous 2-D or 3-D tensor into a new contiguous tensor."""
    assert x.is_contiguous() and x.dim() in (2, 3)
    batch = x.shape[0] if x.dim() == 3 else 1
    R, Cc = x.shape[-2], x.shape[-1]
    out = torch.empty(x.shape[:-2] + (Cc, R), dtype=x.dtype, device=x.device)
    _lib.check(_lib.load().cueq_transpose(_CODE[x.dtype], batch, R, Cc, x.data_ptr(), out.data_ptr(), _stream(x)), "cueq_transpose")
    return out


def layer_norm_fwd(x: torch.Tensor, gamma, beta, eps: float):
    rows, D = x.shape
    y = torch.empty_like(x)
    mean = torch.empty(rows, dtype=torch.float32, device=x.device)
    rstd = torch.empty(rows, dtype=torch.float32, device=x.device)
    _lib.check(
        _lib.load().cueq_layer_norm_fwd(_CODE[x.dtype], rows, D, x.data_ptr(), _ptr(gamma), _ptr(beta), float(eps), y.data_ptr(),
                                        mean.data_ptr(), rstd.data_ptr(), _stream(x)),
        "cueq_layer_norm_fwd",
    )
    return y, mean, rstd


def layer_norm_bwd(dy: torch.Tensor, x: torch.Tensor, mean, rstd, gamma, need_affine: bool):
    rows, D = x.shape
    lib = _lib.load()
    dx = torch.empty_like(x)
    dgamma = torch.empty(D, dtype=torch.float32, device=x.device) if need_affine else None
    dbeta = torch.empty(D, dtype=torch.float32, device=x.device) if need_affine else None
    ws_bytes = lib.cueq_layer_norm_bwd_workspace(rows, D)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=x.device)
    _lib.check(
        lib.cueq_layer_norm_bwd(_CODE[x.dtype], rows, D, dy.data_ptr(), x.data_ptr(), mean.data_ptr(), rstd.data_ptr(), _ptr(gamma),
                                dx.data_ptr(), _ptr(dgamma), _ptr(dbeta), ws.data_ptr(), ws_bytes, _stream(x)),
        "cueq_layer_norm_bwd",
    )
    return dx, dgamma, dbeta


def _ln_t_ok(xt: torch.Tensor) -> bool:
    D, M = xt.shape
    epv = 16 // xt.element_size()
    return D <= 256 and D % epv == 0 and M % epv == 0 and xt.data_ptr() % 16 == 0


def layer_norm_t_fwd(xt: torch.Tensor, gamma, beta, eps: float):
    """LayerNorm over d of ``xt (D, M)`` into ``y (M, D)`` (one kernel, no transposed copy)."""
    D, M = xt.shape
    y = torch.empty(M, D, dtype=xt.dtype, device=xt.device)
    mean = torch.empty(M, dtype=torch.float32, device=xt.device)
    rstd = torch.empty(M, dtype=torch.float32, device=xt.device)
    _lib.check(
        _lib.load().cueq_layer_norm_t_fwd(_CODE[xt.dtype], M, D, xt.data_ptr(), _ptr(gamma), _ptr(beta), float(eps), y.data_ptr(),
                                          mean.data_ptr(), rstd.data_ptr(), _stream(xt)),
        "cueq_layer_norm_t_fwd",
    )
    return y, mean, rstd


def layer_norm_t_bwd(dy: torch.Tensor, xt: torch.Tensor, mean, rstd, gamma, need_affine: bool):
    """Backward of :func:`layer_norm_t_fwd`: ``dy (M, D)`` -> ``dxt (D, M)`` (+ float32 ``dgamma``, ``dbeta``)."""
    D, M = xt.shape
    lib = _lib.load()
    dxt = torch.empty_like(xt)
    dgamma = torch.empty(D, dtype=torch.float32, device=xt.device) if need_affine else None
    dbeta = torch.empty(D, dtype=torch.float32, device=xt.device) if need_affine else None
    ws_bytes = lib.cueq_layer_norm_t_bwd_workspace(_CODE[xt.dtype], M, D) if need_affine else 0
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=xt.device) if need_affine else None
    _lib.check(
        lib.cueq_layer_norm_t_bwd(_CODE[xt.dtype], M, D, dy.data_ptr(), xt.data_ptr(), mean.data_ptr(), rstd.data_ptr(), _ptr(gamma),
                                  dxt.data_ptr(), _ptr(dgamma), _ptr(dbeta), _ptr(ws), ws_bytes, _stream(xt)),
        "cueq_layer_norm_t_bwd",
    )
    return dxt, dgamma, dbeta


def gate_fwd(u, v, bias_u, bias_v, bias_axis: int, mask, mask_axis: int, dtype) -> torch.Tensor:
    rows, cols = u.shape
    out = torch.empty(rows, cols, dtype=dtype, device=u.device)
    _lib.check(
        _lib.load().cueq_gate_fwd(_CODE[dtype], rows, cols, u.data_ptr(), v.data_ptr(), _ptr(bias_u), _ptr(bias_v), bias_axis,
                                  _ptr(mask), mask_axis, out.data_ptr(), _stream(u)),
        "cueq_gate_fwd",
    )
    return out


def gate_bwd(dout, u, v, bias_u, bias_v, bias_axis: int, mask, mask_axis: int):
    rows, cols = u.shape
    du, dv = torch.empty_like(dout), torch.empty_like(dout)
    _lib.check(
        _lib.load().cueq_gate_bwd(_CODE[dout.dtype], rows, cols, dout.data_ptr(), u.data_ptr(), v.data_ptr(), _ptr(bias_u),
                                  _ptr(bias_v), bias_axis, _ptr(mask), mask_axis, du.data_ptr(), dv.data_ptr(), _stream(u)),
        "cueq_gate_bwd",
    )
    return du, dv


def _fusable(*tensors) -> bool:
    """The fused projection + gate kernel moves 16-byte vectors: row strides and addresses must allow it."""
    for t in tensors:
        if t is None:
            continue
        if t.data_ptr() % 16 or (t.dim() == 2 and (t.stride(0) * t.element_size()) % 16):
            return False
    return True


def dual_gate_fwd(A1, A2, B1, B2, bias1, bias2, bias_axis: int, mask, mask_axis: int) -> torch.Tensor:
    """``sigmoid(A1 B1^T + bias1) * (A2 B2^T + bias2) * mask`` (``B2 is None``: same as ``B1``); the two products stay
    in registers when the operands allow the fused kernel, otherwise they go through float32 buffers."""
    M, K = A1.shape
    N = B1.shape[0]
    T = A1.dtype
    if _fusable(A1, A2, B1, B2) and (K * A1.element_size()) % 16 == 0:
        out = torch.empty(M, N, dtype=T, device=A1.device)
        _lib.check(
            _lib.load().cueq_dual_gate(_CODE[T], 0, M, N, K, A1.data_ptr(), A2.data_ptr(), A1.stride(0), B1.data_ptr(), _ptr(B2),
                                       B1.stride(0), _ptr(bias1), _ptr(bias2), bias_axis, _ptr(mask), mask_axis, None,
                                       out.data_ptr(), None, N, _stream(A1)),
            "cueq_dual_gate",
        )
        return out
    u = gemm_nt(A1, B1, torch.float32)
    v = gemm_nt(A2, B1 if B2 is None else B2, torch.float32)
    return gate_fwd(u, v, bias1, bias2, bias_axis, mask, mask_axis, T)


def ln_dual_gate_fwd(x, gamma, beta, eps: float, W1, W2, bias1, bias2, mask):
    """``LayerNorm`` of the rows of ``x (M, K)`` and ``sigmoid(W1 xh^T + bias1) * (W2 xh^T + bias2) * mask`` in one kernel
    (``cueq_ln_dual_gate``).  Returns ``(out (C, M), xh, mean, rstd)``, or ``None`` when the shapes do not allow it
    (then :func:`layer_norm_fwd` and :func:`dual_gate_fwd` do the same in two launches)."""
    M, K = x.shape
    Cn = W1.shape[0]
    if x.dtype not in _TWO_BYTE or K % 32 or K > 128 or Cn % 32 or M % 2 or M < 4096 or M > 65280 * 128:
        return None
    if 2 * Cn * (2 * K if K == 128 else 2 * K + 16) + 8 * Cn + 8 * K > 160 * 1024 or not _fusable(x, W1, W2):
        return None
    out = torch.empty(Cn, M, dtype=x.dtype, device=x.device)
    xh = torch.empty(M, K, dtype=x.dtype, device=x.device)
    mean = torch.empty(M, dtype=torch.float32, device=x.device)
    rstd = torch.empty(M, dtype=torch.float32, device=x.device)
    _lib.check(
        _lib.load().cueq_ln_dual_gate(_CODE[x.dtype], Cn, M, K, W1.data_ptr(), W2.data_ptr(), W1.stride(0), x.data_ptr(), x.stride(0),
                                      _ptr(gamma), _ptr(beta), float(eps), _ptr(bias1), _ptr(bias2), _ptr(mask), out.data_ptr(), M,
                                      xh.data_ptr(), K, mean.data_ptr(), rstd.data_ptr(), _stream(x)),
        "cueq_ln_dual_gate",
    )
    return out, xh, mean, rstd


def dual_gate_bwd(dout, A1, A2, B1, B2, bias1, bias2, bias_axis: int, mask, mask_axis: int):
    """Gradients of the two products of :func:`dual_gate_fwd` (they are recomputed, not read back)."""
    M, K = A1.shape
    N = B1.shape[0]
    T = A1.dtype
    if _fusable(A1, A2, B1, B2, dout) and (K * A1.element_size()) % 16 == 0:
        du, dv = torch.empty(M, N, dtype=T, device=A1.device), torch.empty(M, N, dtype=T, device=A1.device)
        _lib.check(
            _lib.load().cueq_dual_gate(_CODE[T], 1, M, N, K, A1.data_ptr(), A2.data_ptr(), A1.stride(0), B1.data_ptr(), _ptr(B2),
                                       B1.stride(0), _ptr(bias1), _ptr(bias2), bias_axis, _ptr(mask), mask_axis, dout.data_ptr(),
                                       du.data_ptr(), dv.data_ptr(), N, _stream(A1)),
            "cueq_dual_gate",
        )
        return du, dv
    u = gemm_nt(A1, B1, torch.float32)
    v = gemm_nt(A2, B1 if B2 is None else B2, torch.float32)
    return gate_bwd(dout, u, v, bias1, bias2, bias_axis, mask, mask_axis)


def gate_bwd_input(dC, dc_by_row: bool, W1, W2, X1, X2, bias1, bias2, mask, dX1=None, want_gate_grads: bool = False):
    """Backward of ``sigmoid(W1 X1^T + b1) * (W2 X2^T + b2) * mask`` (rows ``c``, columns ``m``) down to ``X1``/``X2``
    in one kernel (``cueq_gate_bwd_input``); ``dC`` is ``(C, M)`` when ``dc_by_row`` else ``(M, C)``.  ``X2 is None``: one
    input, whose gradient is added to ``dX1`` when that is given.  Returns ``(dX1, dX2, dU, dV)`` (``dU, dV`` in the layout
    of ``dC``, only when ``want_gate_grads``), or ``None`` when the shapes do not allow the fused kernel."""
    Cn, K = W1.shape
    M = X1.shape[0]
    T = W1.dtype
    es = W1.element_size()
    if K % 32 or K > 128 or Cn % 32 or not _fusable(W1, W2, X1, X2, dC, dX1):
        return None
    accumulate = dX1 is not None
    if dX1 is None:
        dX1 = torch.empty(M, K, dtype=T, device=W1.device)
    dX2 = torch.empty(M, K, dtype=T, device=W1.device) if X2 is not None else None
    dU = torch.empty_like(dC) if want_gate_grads else None
    dV = torch.empty_like(dC) if want_gate_grads else None
    _lib.check(
        _lib.load().cueq_gate_bwd_input(_CODE[T], Cn, M, K, W1.data_ptr(), W2.data_ptr(), W1.stride(0),
                                        X1.data_ptr(), _ptr(X2), X1.stride(0), _ptr(bias1), _ptr(bias2), _ptr(mask), dC.data_ptr(),
                                        dC.stride(0), int(dc_by_row), dX1.data_ptr(), _ptr(dX2), dX1.stride(0), int(accumulate),
                                        _ptr(dU), _ptr(dV), _stream(W1)),
        "cueq_gate_bwd_input",
    )
    return dX1, dX2, dU, dV


def gate_bwd_input_ln(dC, W1, W2, X, bias1, bias2, mask, dX, ln_x, ln_mean, ln_rstd, ln_gamma):
    """:func:`gate_bwd_input` in its one-input form (``dC`` is ``(C, M)``) continued through the LayerNorm that produced ``X``
    from ``ln_x``, in one kernel (``cueq_gate_bwd_input_ln``): ``dX`` (the gradient that has already arrived at ``X``, or
    ``None``) is replaced by the gradient with respect to ``ln_x``.  Returns it, or ``None`` when the shapes do not allow the
    kernel (then :func:`gate_bwd_input` and :func:`layer_norm_bwd` do the same in two launches)."""
    Cn, K = W1.shape
    M = X.shape[0]
    T = W1.dtype
    if T not in _TWO_BYTE or K % 32 or K > 128 or Cn % 32 or M % 2 or dC.stride(0) % 2 or dC.data_ptr() % 4:
        return None
    if 2 * Cn * (2 * K if K == 128 else 2 * K + 16) + 8 * Cn + 4 * K > 160 * 1024 or not _fusable(W1, W2, X, dX, ln_x):
        return None
    if (4 * dC.stride(0) + M) * 2 >= (1 << 32) or M >= (1 << 31) - 128:
        return None
    accumulate = dX is not None
    if dX is None:
        dX = torch.empty(M, K, dtype=T, device=W1.device)
    _lib.check(
        _lib.load().cueq_gate_bwd_input_ln(_CODE[T], Cn, M, K, W1.data_ptr(), W2.data_ptr(), W1.stride(0), X.data_ptr(), X.stride(0),
                                           _ptr(bias1), _ptr(bias2), _ptr(mask), dC.data_ptr(), dC.stride(0), dX.data_ptr(), dX.stride(0),
                                           int(accumulate), ln_x.data_ptr(), ln_x.stride(0), ln_mean.data_ptr(), ln_rstd.data_ptr(),
                                           _ptr(ln_gamma), _stream(W1)),
        "cueq_gate_bwd_input_ln",
    )
    return dX


def sum_cols(x: torch.Tensor) -> torch.Tensor:
    rows, cols = x.shape
    out = torch.empty(rows, dtype=torch.float32, device=x.device)
    _lib.check(_lib.load().cueq_sum_cols(_CODE[x.dtype], rows, cols, x.data_ptr(), out.data_ptr(), _stream(x)), "cueq_sum_cols")
    return out


def sum_rows(x: torch.Tensor) -> torch.Tensor:
    rows, cols = x.shape
    lib = _lib.load()
    out = torch.empty(cols, dtype=torch.float32, device=x.device)
    ws_bytes = lib.cueq_sum_rows_workspace(rows, cols)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=x.device)
    _lib.check(lib.cueq_sum_rows(_CODE[x.dtype], rows, cols, x.data_ptr(), out.data_ptr(), ws.data_ptr(), ws_bytes, _stream(x)), "cueq_sum_rows")
    return out


def _split_k_chunks(K: int, align: int) -> int:
    """Number of equal chunks (each a multiple of ``align``) to split a long contraction into."""
    for n in range(min(512, max(1, K // 512)), 1, -1):
        if K % n == 0 and (K // n) % align == 0:
            return n
    return 1


def gemm_long_k(A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
    """``A (P, K) @ B (Q, K)^T`` in float32 for a very long ``K``: equal k-chunks as a batched GEMM, then an ordered
    sum of the partial products (no atomics)."""
    P, K = A.shape
    Q = B.shape[0]
    n = _split_k_chunks(K, 8 if A.dtype in _TWO_BYTE else 4)
    if n == 1:
        return gemm_nt(A, B, torch.float32)
    ck = K // n
    Ab = A.as_strided((n, P, ck), (ck, A.stride(0), 1))
    Bb = B.as_strided((n, Q, ck), (ck, B.stride(0), 1))
    part = gemm_nt(Ab, Bb, torch.float32)
    return sum_rows(part.view(n, P * Q)).view(P, Q)


# ---------------------------------------------------------------------------------------------
# autograd
# ---------------------------------------------------------------------------------------------
def _trimul_fwd(x, mask, nin_w, nin_b, p_in_w, p_in_b, g_in_w, g_in_b, nout_w, nout_b, p_out_w, p_out_b, g_out_w, g_out_b,
                outgoing: bool, eps: float):
    """Forward of the update on ``x (B, N, N, D)``: returns the output, the tensors the backward reads (inputs first,
    then the eight computed ones) and the extents."""
    if True:
        T = x.dtype
        Bsz, N, _, D = x.shape
        M = Bsz * N * N
        Do = p_out_w.shape[0]
        x2 = x.reshape(M, D)
        mflat = None if mask is None else mask.reshape(M)
        # (2D, M) == (2D, B, N, N): the "transposed output" of the reference comes for free with the weights as rows
        fused = ln_dual_gate_fwd(x2, nin_w, nin_b, eps, g_in_w, p_in_w, g_in_b, p_in_b, mflat)
        if fused is not None:
            ab, xh, mean1, rstd1 = fused
        else:
            xh, mean1, rstd1 = layer_norm_fwd(x2, nin_w, nin_b, eps)
            ab = dual_gate_fwd(g_in_w, p_in_w, xh, None, g_in_b, p_in_b, 0, mflat, 1)
        a = ab[:D].view(D * Bsz, N, N)
        b = ab[D:].view(D * Bsz, N, N)
        if outgoing:
            t = gemm_nt(a, b, T)  # t[i, j] = sum_k a[i, k] b[j, k]
        else:
            t = gemm_nt(a, b, T, trans_a=True, trans_b=True)  # t[i, j] = sum_k a[k, i] b[k, j]
        t2 = t.view(D, M)
        if _ln_t_ok(t2):
            y, mean2, rstd2 = layer_norm_t_fwd(t2, nout_w, nout_b, eps)  # (M, D)
        else:
            y, mean2, rstd2 = layer_norm_fwd(transpose(t2), nout_w, nout_b, eps)
        out = dual_gate_fwd(xh, y, g_out_w, p_out_w, g_out_b, p_out_b, 1, None, 0)  # (M, Do)
        saved = (x2, mflat, nin_w, p_in_w, p_in_b, g_in_w, g_in_b, nout_w, p_out_w, p_out_b, g_out_w, g_out_b,
                 xh, mean1, rstd1, ab, t2, mean2, rstd2, y)
        has = (nin_w is not None, nin_b is not None, nout_w is not None, nout_b is not None)
        return out.view(Bsz, N, N, Do), saved, (Bsz, N, D, Do), has


def _cast(g, like, have):
    return g.to(like.dtype) if (g is not None and have) else None


def _trimul_bwd(saved, dims, has, outgoing: bool, need, dout):
    """Gradients for the 16 arguments of :func:`_trimul_fwd` (``need[k]``: whether argument ``k`` wants one)."""
    if True:
        (x2, mflat, nin_w, p_in_w, p_in_b, g_in_w, g_in_b, nout_w, p_out_w, p_out_b, g_out_w, g_out_b,
         xh, mean1, rstd1, ab, t2, mean2, rstd2, y) = saved
        Bsz, N, D, Do = dims
        M = Bsz * N * N
        T = x2.dtype
        dout = dout.contiguous().view(M, Do).to(T)

        # output gate
        w_out = need[10] or need[11] or need[12] or need[13]
        fused = gate_bwd_input(dout, False, g_out_w, p_out_w, xh, y, g_out_b, p_out_b, None, None, w_out)
        if fused is not None:
            dxh, dy, du2, dv2 = fused
        else:
            du2, dv2 = dual_gate_bwd(dout, xh, y, g_out_w, p_out_w, g_out_b, p_out_b, 1, None, 0)  # (M, Do)
            dxh = gemm_nt(du2, transpose(g_out_w), T)  # (M, D)
            dy = gemm_nt(dv2, transpose(p_out_w), T)
        w_in = need[4] or need[5] or need[6] or need[7]
        xhT = transpose(xh) if (w_in or need[12]) else None  # (D, M)
        d_g_out_w = d_p_out_w = d_g_out_b = d_p_out_b = None
        if need[12]:
            d_g_out_w = gemm_long_k(transpose(du2), xhT).to(g_out_w.dtype)
        if need[10]:
            d_p_out_w = gemm_long_k(transpose(dv2), transpose(y)).to(p_out_w.dtype)
        if g_out_b is not None and need[13]:
            d_g_out_b = sum_rows(du2).to(g_out_b.dtype)
        if p_out_b is not None and need[11]:
            d_p_out_b = sum_rows(dv2).to(p_out_b.dtype)

        # LayerNorm across d
        affine_out = (has[2] and need[8]) or (has[3] and need[9])
        if _ln_t_ok(t2):
            dt, d_nout_w, d_nout_b = layer_norm_t_bwd(dy, t2, mean2, rstd2, nout_w, affine_out)  # (D, M)
        else:
            dtT, d_nout_w, d_nout_b = layer_norm_bwd(dy, transpose(t2), mean2, rstd2, nout_w, affine_out)
            dt = transpose(dtT)
        dt = dt.view(D * Bsz, N, N)  # (D, M) viewed per (d, b)

        # triangular contraction
        a = ab[:D].view(D * Bsz, N, N)
        b = ab[D:].view(D * Bsz, N, N)
        dab = torch.empty_like(ab)
        da = dab[:D].view(D * Bsz, N, N)
        db = dab[D:].view(D * Bsz, N, N)
        if outgoing:  # t = a b^T
            gemm_nt(dt, b, T, out=da, trans_b=True)  # da[i, k] = sum_j dt[i, j] b[j, k]
            gemm_nt(dt, a, T, out=db, trans_a=True, trans_b=True)  # db[j, k] = sum_i dt[i, j] a[i, k]
        else:  # t = a^T b
            gemm_nt(b, dt, T, out=da)  # da[k, i] = sum_j b[k, j] dt[i, j]
            gemm_nt(a, dt, T, out=db, trans_b=True)  # db[k, j] = sum_i a[k, i] dt[i, j]

        # input gate and projections - and, when neither their weights nor the LayerNorm's ask for a gradient, the input
        # LayerNorm in the same kernel
        affine_in = (has[0] and need[2]) or (has[1] and need[3])
        if not w_in and not affine_in and need[0]:
            dx = gate_bwd_input_ln(dab, g_in_w, p_in_w, xh, g_in_b, p_in_b, mflat, dxh, x2, mean1, rstd1, nin_w)
            if dx is not None:
                return (dx.view(Bsz, N, N, D), None, None, None, None, None, None, None, _cast(d_nout_w, x2, has[2]), _cast(d_nout_b, x2, has[3]),
                        d_p_out_w, d_p_out_b, d_g_out_w, d_g_out_b, None, None)
        fused = gate_bwd_input(dab, True, g_in_w, p_in_w, xh, None, g_in_b, p_in_b, mflat, dxh, w_in)
        if fused is not None:
            du1, dv1 = fused[2], fused[3]
        else:
            du1, dv1 = dual_gate_bwd(dab, g_in_w, p_in_w, xh, None, g_in_b, p_in_b, 0, mflat, 1)  # (2D, M)
            gemm_nt(transpose(du1), transpose(g_in_w), T, out=dxh, accumulate=True)
            gemm_nt(transpose(dv1), transpose(p_in_w), T, out=dxh, accumulate=True)
        d_g_in_w = d_p_in_w = d_g_in_b = d_p_in_b = None
        if need[6]:
            d_g_in_w = gemm_long_k(du1, xhT).to(g_in_w.dtype)
        if need[4]:
            d_p_in_w = gemm_long_k(dv1, xhT).to(p_in_w.dtype)
        if g_in_b is not None and need[7]:
            d_g_in_b = sum_cols(du1).to(g_in_b.dtype)
        if p_in_b is not None and need[5]:
            d_p_in_b = sum_cols(dv1).to(p_in_b.dtype)

        # input LayerNorm
        dx, d_nin_w, d_nin_b = layer_norm_bwd(dxh, x2, mean1, rstd1, nin_w, affine_in)
        dx = dx.view(Bsz, N, N, D) if need[0] else None
        return (dx, None, _cast(d_nin_w, x2, has[0]), _cast(d_nin_b, x2, has[1]), d_p_in_w, d_p_in_b, d_g_in_w, d_g_in_b,
                _cast(d_nout_w, x2, has[2]), _cast(d_nout_b, x2, has[3]), d_p_out_w, d_p_out_b, d_g_out_w, d_g_out_b, None, None)


class _TriMul(torch.autograd.Function):
    @staticmethod
    def forward(ctx, *args):
        out, saved, dims, has = _trimul_fwd(*args)
        ctx.save_for_backward(*saved)
        ctx.outgoing, ctx.dims, ctx.has = args[14], dims, has
        return out

    @staticmethod
    def backward(ctx, dout):
        return _trimul_bwd(ctx.saved_tensors, ctx.dims, ctx.has, ctx.outgoing, ctx.needs_input_grad, dout)


# ---------------------------------------------------------------------- traced execution (torch.compile / export)
# Two opaque operators, forward and backward, around the same two functions.  Optional tensors travel as empty
# placeholders plus a presence list (operator schemas have no optional entries inside tensor lists; the list holds
# integers because torch.jit.trace does not take lists of booleans).
def _placeholders(ref: torch.Tensor, tensors):
    return [ref.new_empty(0) if t is None else t for t in tensors], [int(t is not None) for t in tensors]


@torch.library.custom_op("cuequivariance_amd::trimul_fwd", mutates_args=(), device_types="cuda")
def _trimul_fwd_op(x: torch.Tensor, tensors: List[torch.Tensor], present: List[int], outgoing: bool, eps: float) -> List[torch.Tensor]:
    args = [t if p else None for t, p in zip(tensors, present)]  # mask, then the 12 weights
    out, saved, _, _ = _trimul_fwd(x, *args, outgoing, eps)
    return [out, *saved[12:]]  # + xh, mean1, rstd1, ab, t2, mean2, rstd2, y


@_trimul_fwd_op.register_fake
def _trimul_fwd_fake(x, tensors, present, outgoing, eps):
    Bsz, N, _, D = x.shape
    M = Bsz * N * N
    Do = tensors[9].shape[0]  # p_out_weight
    f32 = dict(dtype=torch.float32)
    return [x.new_empty(Bsz, N, N, Do), x.new_empty(M, D), x.new_empty(M, **f32), x.new_empty(M, **f32), x.new_empty(2 * D, M),
            x.new_empty(D, M), x.new_empty(M, **f32), x.new_empty(M, **f32), x.new_empty(M, D)]


@torch.library.custom_op("cuequivariance_amd::trimul_bwd", mutates_args=(), device_types="cuda")
def _trimul_bwd_op(dout: torch.Tensor, x: torch.Tensor, tensors: List[torch.Tensor], computed: List[torch.Tensor], present: List[int],
                   need: List[bool], outgoing: bool) -> List[torch.Tensor]:
    mask, nin_w, nin_b, p_in_w, p_in_b, g_in_w, g_in_b, nout_w, nout_b, p_out_w, p_out_b, g_out_w, g_out_b = [
        t if p else None for t, p in zip(tensors, present)]
    Bsz, N, _, D = x.shape
    M = Bsz * N * N
    saved = (x.reshape(M, D), None if mask is None else mask.reshape(M), nin_w, p_in_w, p_in_b, g_in_w, g_in_b, nout_w, p_out_w, p_out_b,
             g_out_w, g_out_b, *computed)
    has = (nin_w is not None, nin_b is not None, nout_w is not None, nout_b is not None)
    grads = _trimul_bwd(saved, (Bsz, N, D, p_out_w.shape[0]), has, outgoing, [*need, False, False], dout)
    return [x.new_empty(0) if (g is None or not n) else g.contiguous() for g, n in zip(grads[:14], need)]


@_trimul_bwd_op.register_fake
def _trimul_bwd_fake(dout, x, tensors, computed, present, need, outgoing):
    like = [x, *tensors]
    return [torch.empty_like(t) if (n and (k == 0 or present[k - 1]) and k != 1) else x.new_empty(0) for k, (t, n) in enumerate(zip(like, need))]


def _trimul_setup_context(ctx, inputs, output):
    x, tensors, present, outgoing, eps = inputs
    ctx.present, ctx.outgoing, ctx.ntensors = list(present), outgoing, len(tensors)
    ctx.save_for_backward(x, *tensors, *output[1:])


def _trimul_autograd(ctx, grads):
    saved = ctx.saved_tensors
    x, tensors, computed = saved[0], list(saved[1: 1 + ctx.ntensors]), list(saved[1 + ctx.ntensors:])
    flags = ctx.needs_input_grad[1]
    if isinstance(flags, bool):
        flags = [flags] * len(tensors)
    need = [bool(ctx.needs_input_grad[0]), *[bool(f) for f in flags]]
    got = _trimul_bwd_op(grads[0], x, tensors, computed, ctx.present, need, ctx.outgoing)
    pick = [g if g.numel() > 0 else None for g in got]
    return pick[0], pick[1:], None, None, None


torch.library.register_autograd("cuequivariance_amd::trimul_fwd", _trimul_autograd, setup_context=_trimul_setup_context)



def _lecun_normal(shape, device, dtype) -> torch.Tensor:
    """Truncated normal with variance 1 / fan_in (the reference's default projection initialiser,
    ``_triangle_multiplicative_update.py:60-96``)."""
    w = torch.empty(shape, device=device, dtype=torch.float32)
    std = math.sqrt(1.0 / shape[1]) / 0.87962566103423978
    torch.nn.init.trunc_normal_(w, mean=0.0, std=std, a=-2.0 * std, b=2.0 * std)
    return w.to(dtype)


def triangle_multiplicative_update(
    x: torch.Tensor,
    direction: str = "outgoing",
    mask: Optional[torch.Tensor] = None,
    norm_in_weight: Optional[torch.Tensor] = None,
    norm_in_bias: Optional[torch.Tensor] = None,
    p_in_weight: Optional[torch.Tensor] = None,
    p_in_bias: Optional[torch.Tensor] = None,
    g_in_weight: Optional[torch.Tensor] = None,
    g_in_bias: Optional[torch.Tensor] = None,
    norm_out_weight: Optional[torch.Tensor] = None,
    norm_out_bias: Optional[torch.Tensor] = None,
    p_out_weight: Optional[torch.Tensor] = None,
    p_out_bias: Optional[torch.Tensor] = None,
    g_out_weight: Optional[torch.Tensor] = None,
    g_out_bias: Optional[torch.Tensor] = None,
    eps: float = 1e-5,
    precision: Optional[TriMulPrecision] = None,
) -> torch.Tensor:
    """Triangle multiplicative update of a pair tensor ``x (..., N, N, D)``; see the module docstring.

    ``mask (..., N, N)`` multiplies the gated projections; norm weights default to 1 / biases to 0, projection
    biases to none; projection weights that are not given are drawn (truncated normal, variance ``1 / D``) at
    every call, as a stand-in for the reference's initialiser - pass them for anything but a shape test.
    ``D`` must be a multiple of 32 (reference ``primitives/triangle.py:207``).  Differentiable with respect to
    ``x`` and every weight given.
    """
    if direction not in ("outgoing", "incoming"):
        raise ValueError("direction must be either 'outgoing' or 'incoming'")
    if precision is not None and not isinstance(precision, (TriMulPrecision, int)):
        raise ValueError("precision must be a TriMulPrecision or None")
    if x.dim() < 3:
        raise ValueError("x must have shape (..., N, N, D)")
    if x.dim() == 3:
        x = x.unsqueeze(0)
        if mask is not None and mask.dim() == 2:
            mask = mask.unsqueeze(0)
    lead = x.shape[:-3]
    N, N2, D = x.shape[-3:]
    if N != N2:
        raise ValueError(f"x must be square in its two sequence dimensions, got {N} x {N2}")
    if D % 32 != 0:
        raise ValueError("hidden dimension must be a multiple of 32")
    if not x.is_cuda:
        raise ValueError("triangle_multiplicative_update runs on the GPU only: x is on " + str(x.device))
    if x.dtype not in _CODE:
        raise ValueError(f"x must be float32, bfloat16 or float16, got {x.dtype}")
    T, dev = x.dtype, x.device
    if mask is not None and tuple(mask.shape) != tuple(lead) + (N, N):
        raise ValueError(f"mask must have shape {tuple(lead) + (N, N)}, got {tuple(mask.shape)}")

    def vec(t, n, name):
        if t is None:
            return None
        if tuple(t.shape) != (n,):
            raise ValueError(f"{name} must have shape ({n},), got {tuple(t.shape)}")
        return t.to(T).contiguous()

    def mat(t, shape, name):
        if t is None:
            with torch.no_grad():
                return _lecun_normal(shape, dev, T)
        if tuple(t.shape) != shape and not (shape[0] is None and t.dim() == 2 and t.shape[1] == shape[1]):
            raise ValueError(f"{name} must have shape {shape}, got {tuple(t.shape)}")
        return t.to(T).contiguous()

    Do = D
    if p_out_weight is not None:
        Do = p_out_weight.shape[0]
    elif g_out_weight is not None:
        Do = g_out_weight.shape[0]
    args = (
        vec(norm_in_weight, D, "norm_in_weight"), vec(norm_in_bias, D, "norm_in_bias"),
        mat(p_in_weight, (2 * D, D), "p_in_weight"), vec(p_in_bias, 2 * D, "p_in_bias"),
        mat(g_in_weight, (2 * D, D), "g_in_weight"), vec(g_in_bias, 2 * D, "g_in_bias"),
        vec(norm_out_weight, D, "norm_out_weight"), vec(norm_out_bias, D, "norm_out_bias"),
        mat(p_out_weight, (Do, D), "p_out_weight"), vec(p_out_bias, Do, "p_out_bias"),
        mat(g_out_weight, (Do, D), "g_out_weight"), vec(g_out_bias, Do, "g_out_bias"),
    )
    Bsz = 1
    for s in lead:
        Bsz *= s
    xf = x.reshape(Bsz, N, N, D).contiguous()
    mf = None if mask is None else mask.reshape(Bsz, N, N).to(T).contiguous()
    if torch.compiler.is_compiling() or torch.jit.is_tracing() or type(xf) not in (torch.Tensor, torch.nn.Parameter):
        tensors, present = _placeholders(xf, [mf, *args])
        out = _trimul_fwd_op(xf, tensors, present, direction == "outgoing", float(eps))[0]
    else:
        out = _TriMul.apply(xf, mf, *args, direction == "outgoing", float(eps))
    return out.view(tuple(lead) + (N, N, Do))
