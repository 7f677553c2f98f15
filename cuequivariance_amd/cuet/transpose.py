"""Layout glue: per-segment ``(u, v) -> (v, u)`` transposition between ``mul_ir`` and ``ir_mul``.

Mirror of ``cuequivariance_torch/cuequivariance_torch/primitives/transpose.py:23-183``.
The descriptors of this package use ``ir_mul``; with ``layout=cue.ir_mul`` these modules
are the identity.  For ``mul_ir`` callers the transposition is done with tensor views on
the device (reshape / transpose / cat), which is what the reference does when its native
transpose op is absent (same file, lines 134-152).
"""

from __future__ import annotations

from typing import Optional

import torch

from .. import cue

__all__ = ["TransposeSegments", "TransposeIrrepsLayout"]


class TransposeSegments(torch.nn.Module):
    def __init__(self, segments: list[tuple[int, int]], device: Optional[torch.device] = None, use_fallback=None):
        super().__init__()
        self.segments = [(int(u), int(v)) for u, v in segments]
        self.trivial = all(u == 1 or v == 1 for u, v in self.segments)

    def __repr__(self):
        return "TransposeSegments()"

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.trivial:
            return x
        outs, off = [], 0
        for u, v in self.segments:
            seg = x[..., off: off + u * v]
            outs.append(seg.reshape(x.shape[:-1] + (u, v)).transpose(-2, -1).reshape(x.shape[:-1] + (u * v,)))
            off += u * v
        return torch.cat(outs, dim=-1)


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

    def __repr__(self):
        return f"TransposeIrrepsLayout({self.source} -> {self.target})"

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.f(x)
