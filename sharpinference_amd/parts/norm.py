"""Normalisation parts."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..ops.profile import section
from .base import INIT_NORM_WEIGHT, ParamSpec, Part, ResidualStream, TensorSource


class RMSNorm(Part):
    """x * rsqrt(mean(x^2) + eps) * w, statistics in float
    (reference: src/SharpInference.Cpu/SimdKernels.cs:4209-4246; CUDA twin
    src/SharpInference.Cuda/CudaTextKernels.cs:199-224).  ``has_weight=False`` is the
    weightless form (SimdKernels.cs:4252-4283).  ``weight_offset`` c: the stored weight lies around
    zero and stands for c + w (the sum is formed once, in float, when the weight is loaded)."""

    def __init__(self, dim: int, eps: float, has_weight: bool = True, name: str = "weight", weight_offset: float = 0.0):
        self.dim, self.eps, self.has_weight = int(dim), float(eps), bool(has_weight)
        self.weight_offset = float(weight_offset)
        self.name = name           # the weight's name behind the part's prefix ("" : the prefix is the name)
        self.weight: Optional[torch.Tensor] = None
        self._weight_f32: Optional[torch.Tensor] = None

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        return {prefix + self.name: ParamSpec((self.dim,), INIT_NORM_WEIGHT)} if self.has_weight else {}

    def load(self, prefix: str, source: TensorSource) -> None:
        if self.has_weight:
            self.weight = source.get(prefix + self.name)
            if self.weight_offset:
                self.weight = (self.weight.float() + self.weight_offset).contiguous()
            self._weight_f32 = None

    def add_normed(self, stream: ResidualStream, delta, out_dtype: Optional[torch.dtype]) -> None:
        """The norm on a branch's output: h += unit_rms(delta) * w in float (delta a tensor or a
        sum of experts' rows still to be formed), and ``stream.act`` = the new h in ``out_dtype``
        (h itself where that is float32: no copy is made)."""
        copy = out_dtype is not None and out_dtype != torch.float32
        with section("norm", nbytes=stream.h.shape[0] * self.dim * 12):
            if isinstance(delta, ops.BranchMean):
                ops.post_pre_norm(stream.h, delta, self.weight_f32(stream.h.device), self.eps)
                out = ops.cast(stream.h, out_dtype) if copy else None
            else:
                out = ops.norm_add(stream.h, delta, self.weight_f32(stream.h.device), self.eps, out_dtype if copy else None)
        stream.act = out if copy else stream.h

    def weight_f32(self, device) -> torch.Tensor:
        if self._weight_f32 is None:
            self._weight_f32 = self.weight.float().contiguous() if self.has_weight else \
                torch.ones(self.dim, dtype=torch.float32, device=device)
        return self._weight_f32

    def after(self, post: "RMSNorm", stream: ResidualStream, delta, out_dtype: torch.dtype) -> torch.Tensor:
        """h += post(delta), then this norm of the new h, in one launch: the norm behind a branch and the
        norm before the next.  delta: a tensor or a join of branches still to be formed."""
        dev = stream.h.device
        if stream.h.shape[1] > ops.POST_PRE_NORM_MAX_WIDTH or post.eps != self.eps or \
                (isinstance(delta, ops.BranchMean) and delta.eps != post.eps) or not isinstance(delta, (torch.Tensor, ops.BranchMean)):
            post.add_normed(stream, delta if isinstance(delta, torch.Tensor) else delta.tensor(), None)
            return self.forward(stream, out_dtype)
        with section("norm", nbytes=stream.h.shape[0] * self.dim * 16):
            return ops.post_pre_norm(stream.h, delta, post.weight_f32(dev), post.eps, self.weight_f32(dev), out_dtype)

    def forward(self, stream: ResidualStream, out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Fold the pending branch output into the residual sum and normalise.  With ``rows``
        only those rows are produced and the stream is left as it is."""
        if stream.pending_norm is not None:
            if rows is None:       # a branch output waits behind a norm of its own: both norms in one launch
                post, delta = stream.pending_norm, stream.pending
                stream.pending = stream.pending_norm = None
                return self.after(post, stream, delta, out_dtype)
            stream.settle()
        if isinstance(stream.pending, ops.BranchSum):      # a scaled sum of branches: added in float, then the norm
            if rows is None:
                with section("norm", nbytes=stream.h.shape[0] * self.dim * (8 + 4 * len(stream.pending.xs))):
                    ops.stream_add(stream.h, stream.pending)
                stream.pending = None
            else:
                stream.pending = stream.pending.tensor()
        n = stream.h.shape[0] if rows is None else rows.shape[0]
        with section("norm", nbytes=n * self.dim * 12):
            out = ops.add_rmsnorm(stream.h, stream.pending, self.weight, self.eps, out_dtype, rows=rows,
                                  write_back=rows is None)
        if rows is None:
            stream.pending = None
        return out
