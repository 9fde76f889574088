"""A second input from the token at the end of a layer, and tensors that several parts share."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..ops.profile import section
from .base import INIT_NORM_WEIGHT, ParamSpec, Part, ResidualStream, StepContext, TensorSource


class SharedTensor(Part):
    """A tensor of the model that several parts read (a table with a slice per layer): the model
    declares and loads it once (``DecoderModel(shared=...)``), the parts hold this object."""

    def __init__(self, name: str, shape, kind: str = "normal"):
        self.name, self.shape, self.kind = name, tuple(int(s) for s in shape), kind
        self.tensor: Optional[torch.Tensor] = None

    def param_specs(self, prefix: str = "") -> Dict[str, ParamSpec]:
        return {prefix + self.name: ParamSpec(self.shape, self.kind)}

    def load(self, prefix: str, source: TensorSource) -> None:
        self.tensor = source.get(prefix + self.name)


class TokenSide(Part):
    """What a layer adds to the residual sum x at its end from the token itself: with e the layer's slice
    (``dim`` columns from ``column``) of the token's row of a side table, g = gelu_tanh(W_gate x) * e,
    y = W_proj g, and x += y / sqrt(mean(y^2) + eps) * w.  The sum it reads is the stream with every
    branch output of the layer added; the norm's statistics, its weight and the addition are float."""

    NAMES = {"gate": "gate", "proj": "proj", "norm": "norm"}

    def __init__(self, hidden: int, dim: int, table: SharedTensor, column: int, norm_eps: float,
                 names: Optional[Dict[str, str]] = None):
        if dim < 1 or column < 0 or column + dim > table.shape[1]:
            raise ValueError("the layer's slice must lie inside the side table's rows")
        self.hidden, self.dim, self.table, self.column, self.eps = int(hidden), int(dim), table, int(column), float(norm_eps)
        self.names = {**self.NAMES, **(names or {})}
        self.w_gate = None
        self.w_proj = None
        self.w_norm: Optional[torch.Tensor] = None

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        n = self.names
        return {prefix + n["gate"]: ParamSpec((self.dim, self.hidden)),
                prefix + n["proj"]: ParamSpec((self.hidden, self.dim)),
                prefix + n["norm"]: ParamSpec((self.hidden,), INIT_NORM_WEIGHT)}

    def load(self, prefix: str, source: TensorSource) -> None:
        n = self.names
        self.w_gate = ops.pack_weight(source.get(prefix + n["gate"]))
        self.w_proj = ops.pack_weight(source.get(prefix + n["proj"]))
        self.w_norm = source.get(prefix + n["norm"]).float().contiguous()

    def forward_on_stream(self, stream: ResidualStream, ctx: StepContext) -> None:
        T = stream.h.shape[0]
        width = 2 if ctx.act_dtype == torch.bfloat16 else 4
        stream.settle()
        delta, stream.pending = stream.pending, None
        if delta is not None and not isinstance(delta, (torch.Tensor, ops.BranchSum)):
            delta = delta.tensor()
        with section("token input", nbytes=T * self.hidden * (16 + 2 * width) + 4 * width * T * self.dim + 2 * width * self.dim * self.hidden,
                     flops=4.0 * T * self.hidden * self.dim):
            x = ops.stream_add(stream.h, delta, ctx.act_dtype)
            gate = ops.linear(x, self.w_gate, ctx.act_dtype)
            g = ops.side_gate(gate, ctx.token_ids, self.table.tensor, self.column)
            y = ops.linear(g, self.w_proj, ctx.act_dtype)
            ops.norm_add(stream.h, y, self.w_norm, self.eps)
        stream.act = None
