"""Layout glue: per-segment ``(u, v) -> (v, u)`` transposition between ``mul_ir`` and ``ir_mul``.

Mirror of ``cuequivariance_torch/cuequivariance_torch/primitives/transpose.py:23-183``.
The descriptors of this package use ``ir_mul``; with ``layout=cue.ir_mul`` these modules
are the identity.  For ``mul_ir`` callers the transposition is one HIP kernel
(``cueq_segmented_transpose``: the row permutation is a table built here once per module and device),
differentiable (the backward applies the inverse permutation).
"""

from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from .. import _lib, cue
from .script import scriptable

__all__ = ["TransposeSegments", "TransposeIrrepsLayout"]


def _permutation(segments) -> np.ndarray:
    """``src[o]``: input position of output element ``o`` when every ``(u, v)`` segment becomes ``(v, u)``."""
    parts, off = [], 0
    for u, v in segments:
        parts.append(off + np.arange(u * v, dtype=np.int64).reshape(u, v).T.reshape(-1))
        off += u * v
    return np.concatenate(parts).astype(np.int32) if parts else np.zeros(0, np.int32)


class _Permute(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, fwd_table, bwd_table):
        ctx.tables = (fwd_table, bwd_table)
        return _run(x, fwd_table)

    @staticmethod
    def backward(ctx, g):
        fwd_table, bwd_table = ctx.tables
        return _Permute.apply(g, bwd_table, fwd_table), None, None


def _run(x: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    if not x.is_cuda:
        raise ValueError("TransposeSegments runs on the GPU only: the tensor is on " + str(x.device))
    total = x.shape[-1]
    x2 = x.reshape(-1, total).contiguous()
    out = torch.empty_like(x2)
    _lib.check(
        _lib.load().cueq_segmented_transpose(x2.element_size(), x2.shape[0], total, table.data_ptr(), x2.data_ptr(), out.data_ptr(),
                                             torch.cuda.current_stream(x.device).cuda_stream),
        "cueq_segmented_transpose",
    )
    return out.view(x.shape)


class TransposeSegments(torch.nn.Module):
    def __init__(self, segments: list[tuple[int, int]], device: Optional[torch.device] = None, use_fallback=None):
        super().__init__()
        if use_fallback:
            raise ValueError("use_fallback=True asks for the PyTorch path, which is not part of this engine")
        self.segments = [(int(u), int(v)) for u, v in segments]
        self.trivial = all(u == 1 or v == 1 for u, v in self.segments)
        self.size = sum(u * v for u, v in self.segments)
        fwd = _permutation(self.segments)
        bwd = np.empty_like(fwd)
        bwd[fwd] = np.arange(fwd.size, dtype=np.int32)  # inverse permutation == the table of the (v, u) segments
        self._host_tables = (fwd, bwd)
        self._tables = {}

    def __repr__(self):
        return "TransposeSegments()"

    def _device_tables(self, device):
        key = (device.type, device.index)
        if key not in self._tables:
            self._tables[key] = tuple(torch.from_numpy(t).to(device) for t in self._host_tables)
        return self._tables[key]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if x.shape[-1] != self.size:
            raise ValueError(f"last dimension must be {self.size}, got {x.shape[-1]}")
        if self.trivial:
            return x
        if x.element_size() not in (2, 4, 8):
            raise ValueError(f"unsupported dtype {x.dtype}")
        fwd, bwd = self._device_tables(x.device)
        return _Permute.apply(x, fwd, bwd)


@scriptable("x")
class TransposeIrrepsLayout(torch.nn.Module):
    """Change the layout of a tensor of the given irreps from ``source`` to ``target``."""

    def __init__(self, irreps: cue.Irreps, *, source: cue.IrrepsLayout, target: cue.IrrepsLayout,
                 device: Optional[torch.device] = None, use_fallback=None):
        super().__init__()
        if (source, target) == (cue.mul_ir, cue.ir_mul):
            self.f = TransposeSegments([(mul, ir.dim) for mul, ir in irreps], device=device)
        elif (source, target) == (cue.ir_mul, cue.mul_ir):
            self.f = TransposeSegments([(ir.dim, mul) for mul, ir in irreps], device=device)
        else:
            self.f = torch.nn.Identity()
        self.source, self.target = source, target
        self.is_identity = isinstance(self.f, torch.nn.Identity)  # callers skip the module call then (see `apply_layout`)

    def __repr__(self):
        return f"TransposeIrrepsLayout({self.source} -> {self.target})"

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.f(x)


def apply_layout(t: TransposeIrrepsLayout, x: torch.Tensor) -> torch.Tensor:
    """``t(x)`` without the two module calls when ``t`` changes nothing (a few microseconds each on the host path of small
    batches)."""
    return x if t.is_identity else t(x)
