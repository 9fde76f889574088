"""The gated linear attention mixer: a matrix-valued state per head instead of a cache of keys."""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

from .. import ops
from ..cache.spec import StateSpec
from ..ops.profile import section
from .base import INIT_NORM_WEIGHT, HostStep, LayerCache, ParamSpec, Part, StepContext, StepPlanner, TensorSource

SEGMENT_FROM_TOKENS = 512     # a step whose longest entry has this many tokens gets the segments' work lists
SEGMENT_UP_TO_BLOCKS = 2048   # ... and a layer walks in segments while whole entries would give fewer blocks than this


class WalkSegments(StepPlanner):
    """The work lists of the segmented walk, made once a step for all layers that walk a state: none
    unless some entry is long (decode steps and short portions are walked whole)."""

    key = "linear attention"

    def plan(self, host: HostStep) -> Tuple[List[np.ndarray], dict]:
        if not host.lens or max(host.lens) < SEGMENT_FROM_TOKENS:
            empty = np.zeros(0, dtype=np.int32)
            return [empty, empty], dict(n_segs=0)
        segs, ents = ops.gla_segments(host.lens, host.cu_tokens)
        return [segs.reshape(-1), ents.reshape(-1)], dict(n_segs=segs.shape[0])

    def attach(self, ctx: StepContext, views: List[torch.Tensor], facts: dict) -> None:
        ctx.extras[self.key] = (views[0], views[1]) if facts["n_segs"] else None


_SEGMENTS = WalkSegments()
WALK_SEGMENTS = _SEGMENTS         # every mixer that walks a state token by token shares the step's one list


class GatedLinearAttention(Part):
    """Linear attention with a decay per key channel.  With h the input, per head (dk key
    channels, dv value channels): q = W_q h * dk^(-1/2), k = W_k h, v = W_v h, and a decay
    alpha = sigmoid(z)^(1/tau) in (0, 1) for every key channel, z = W_a2 (W_a1 h) + b through a
    narrow middle (``decay_rank``; in steps of few tokens W_a2, the bias and the decay itself are
    one kernel).  The state S [dk, dv] starts at zero and moves token by token,
    S_t = diag(alpha_t) S_(t-1) + k_t v_t^T; the head's output is o_t = S_t^T q_t, RMS-normed over
    dv with learned weights shared by the heads; the heads side by side are multiplied by
    silu(W_g h) and projected by W_o.

    What is kept per request is the state alone, heads x dk x dv floats in the request's state
    slot (laid out column slice by column slice, ``ops.gla_state_shape``): no pages.  Decays (their logarithm, the division by tau, the exponential), the state and
    the norm are float whatever the activations are stored as.  A step walks each entry's tokens
    in order from the slot's state (csrc/linear_attention.hip), so the outputs of a token do not
    depend on how its request was cut into steps."""

    FUSED_DECAY_TOKENS = 64    # up to so many tokens a step, W_a2, the bias and the decay are one kernel
    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "a1": "a1", "a2": "a2", "a2_bias": "a2.b"}

    def __init__(self, hidden: int, num_heads: int, key_dim: int, value_dim: int, tau: float, decay_rank: int,
                 norm_eps: float, gate: bool = True, names: Optional[Dict[str, str]] = None):
        if min(num_heads, key_dim, value_dim, decay_rank) < 1:
            raise ValueError("heads, key_dim, value_dim and decay_rank must be positive")
        if key_dim > ops.GLA_MAX_KEY_DIM:
            raise ValueError(f"{key_dim} key channels a head are not taken: at most {ops.GLA_MAX_KEY_DIM}")
        if not tau > 0:
            raise ValueError("tau must be positive")
        self.hidden, self.nh, self.dk, self.dv = int(hidden), int(num_heads), int(key_dim), int(value_dim)
        self.tau, self.rank, self.eps, self.has_gate = float(tau), int(decay_rank), float(norm_eps), bool(gate)
        self.names = {**self.NAMES, **(names or {})}
        self.graph_safe = True         # entries and their state slots are read from the step's device arrays
        self.w_in = None               # [q | k | v | g] rows: one product of the input
        self.w_a1 = None               # (a product of its own: a few rows more spoil the large product's shape)
        self.w_a2: Optional[torch.Tensor] = None      # float32 [heads * dk, rank], row-major
        self.b_a2: Optional[torch.Tensor] = None      # float32 [heads * dk]
        self.w_norm: Optional[torch.Tensor] = None    # float32 [dv]
        self.w_o = None

    def step_planners(self):
        return (_SEGMENTS,)

    def cache_spec(self) -> StateSpec:
        return StateSpec(ops.gla_state_shape(self.nh, self.dk, self.dv), torch.float32)

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        n, qk, vv = self.names, self.nh * self.dk, self.nh * self.dv
        specs = {
            prefix + n["q"]: ParamSpec((qk, self.hidden)),
            prefix + n["k"]: ParamSpec((qk, self.hidden)),
            prefix + n["v"]: ParamSpec((vv, self.hidden)),
            prefix + n["o"]: ParamSpec((self.hidden, vv)),
            prefix + n["norm"]: ParamSpec((self.dv,), INIT_NORM_WEIGHT),
            prefix + n["a1"]: ParamSpec((self.rank, self.hidden)),
            prefix + n["a2"]: ParamSpec((qk, self.rank)),
            prefix + n["a2_bias"]: ParamSpec((qk,)),
        }
        if self.has_gate:
            specs[prefix + n["g"]] = ParamSpec((vv, self.hidden))
        return specs

    def load(self, prefix: str, source: TensorSource) -> None:
        n = self.names
        parts = [source.get(prefix + n[k]) for k in (("q", "k", "v", "g") if self.has_gate else ("q", "k", "v"))]
        dt = torch.float32 if any(p.dtype == torch.float32 for p in parts) else parts[0].dtype
        fused = torch.empty(sum(p.shape[0] for p in parts), self.hidden, dtype=dt, device=parts[0].device)
        o = 0
        for p in parts:
            fused[o:o + p.shape[0]].copy_(p)
            o += p.shape[0]
        self.w_in = ops.pack_weight(fused)
        self.w_a1 = ops.pack_weight(source.get(prefix + n["a1"]))
        # the second decay matrix in float whatever the activations are stored as: the decays' logits are then
        # float sums over float values (a narrow middle rounded to bfloat16 would shift every decay of a token)
        self.w_a2 = source.get(prefix + n["a2"]).float().contiguous()
        self.b_a2 = source.get(prefix + n["a2_bias"]).float().contiguous()
        self.w_norm = source.get(prefix + n["norm"]).float().contiguous()
        self.w_o = ops.pack_weight(source.get(prefix + n["o"]))

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        if not cache.write:
            raise ValueError("a recurrent mixer's state cannot be shared between layers")
        T = x.shape[0]
        qk, vv = self.nh * self.dk, self.nh * self.dv
        width = 2 if ctx.act_dtype == torch.bfloat16 else 4
        n_in = 2 * qk + (2 if self.has_gate else 1) * vv
        with section("q|k|v|g", nbytes=width * n_in * (self.hidden + T) + width * T * self.hidden, flops=2.0 * T * self.hidden * n_in):
            proj = ops.linear(x, self.w_in, ctx.act_dtype)
        with section("decays", nbytes=width * self.rank * (self.hidden + T + qk) + 4 * T * qk, flops=2.0 * T * self.rank * (self.hidden + qk)):
            a1 = ops.linear(x, self.w_a1, torch.float32)
            if T <= self.FUSED_DECAY_TOKENS and self.rank <= ops.GLA_FUSED_DECAY_MAX_RANK:
                alpha = ops.gla_decays_from_middle(a1, 0, self.rank, self.w_a2, self.b_a2, self.tau)     # few tokens: one kernel
            else:
                alpha = ops.gla_decays(ops.linear(a1, self.w_a2, torch.float32), self.b_a2, self.tau)
        state = cache.states[0] if cache.states else cache.state
        with section("recurrence", nbytes=lambda: 8 * ctx.n_entries * qk * self.dv + T * (width * (2 * qk + vv) + 4 * (qk + vv)),
                     flops=4.0 * T * qk * self.dv):
            # a long entry alone in its step: walked in segments side by side (twice the sums on many times the blocks)
            whole_blocks = ctx.n_entries * self.nh * ((self.dv + ops.GLA_STATE_COLS - 1) // ops.GLA_STATE_COLS)
            segments = ctx.extras.get(_SEGMENTS.key) if whole_blocks < SEGMENT_UP_TO_BLOCKS else None
            o = ops.gla_walk(proj, 0, qk, 2 * qk, alpha, self.dk ** -0.5, state, ctx, self.nh, self.dk, self.dv, segments=segments)
        with section("head norm + gate", nbytes=T * vv * (4 + 2 * width)):
            y = ops.head_norm_gate(o, self.w_norm, self.eps, self.nh, self.dv, ctx.act_dtype,
                                   proj if self.has_gate else None, 2 * qk + vv)
        with section("o", nbytes=width * self.hidden * (vv + T) + width * T * vv, flops=2.0 * T * self.hidden * vv):
            return ops.linear(y, self.w_o, ctx.act_dtype)
