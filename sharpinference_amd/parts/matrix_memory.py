"""Recurrent mixers whose state is a matrix per head with one scalar decay per token: a matrix memory
with exponential gates, a selective state space behind a short convolution, and retention (a fixed
decay per head)."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..cache.spec import MixedSpec, StateSpec
from ..ops.profile import section
from .base import INIT_NORM_WEIGHT, LayerCache, ParamSpec, Part, StepContext, TensorSource
from .linear_attention import SEGMENT_UP_TO_BLOCKS, WALK_SEGMENTS


def _fuse(parts, hidden: int) -> torch.Tensor:
    dt = torch.float32 if any(p.dtype == torch.float32 for p in parts) else parts[0].dtype
    fused = torch.empty(sum(p.shape[0] for p in parts), hidden, dtype=dt, device=parts[0].device)
    o = 0
    for p in parts:
        fused[o:o + p.shape[0]].copy_(p)
        o += p.shape[0]
    return fused


def _segments_for(ctx: StepContext, nh: int, dv: int):
    """The step's segment lists where a walk of whole entries would leave the chip idle (a long entry alone
    in its step), else None."""
    whole_blocks = ctx.n_entries * nh * ((dv + ops.WALK_STATE_COLS - 1) // ops.WALK_STATE_COLS)
    return ctx.extras.get(WALK_SEGMENTS.key) if whole_blocks < SEGMENT_UP_TO_BLOCKS else None


class MatrixMemory(Part):
    """A matrix memory with exponential gates (the mLSTM cell of xLSTM).  With h the input, per head
    (dk key channels, dv value channels): q = W_q h * dk^(-1/2), k = W_k h, v = W_v h, a log input gate
    i = cap tanh((W_i h + b_i) / cap) and a log forget gate f = log_sigmoid(cap tanh((W_f h + b_f) / cap)).
    A running maximum m_t = max(f_t + m_(t-1), i_t), m_0 = 0, keeps the exponentials in range:
    S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T, n_t likewise with k_t alone, and the
    head's output is S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6), divided by its root mean square
    over dv; the heads side by side times a learned weight per channel, times sigmoid(W_g h), then W_o.

    What is kept per request is S, n and m in its state slot (``ops.walk_state_shape``): no pages.
    The gates' pre-activations are a product of their own with a float result; the gates, the
    maximum, the state, the normaliser and the norm are float whatever the activations are stored
    as.  A step walks each entry's tokens in order from the slot's state (csrc/state_walk.hip)."""

    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "i": "i", "i_bias": "i.b", "f": "f", "f_bias": "f.b"}

    def __init__(self, hidden: int, num_heads: int, key_dim: int, value_dim: int, gate_cap: float, norm_eps: float,
                 names: Optional[Dict[str, str]] = None):
        if min(num_heads, key_dim, value_dim) < 1:
            raise ValueError("heads, key_dim and value_dim must be positive")
        if key_dim > ops.WALK_MAX_KEY_DIM:
            raise ValueError(f"{key_dim} key channels a head are not taken: at most {ops.WALK_MAX_KEY_DIM}")
        if not gate_cap > 0:
            raise ValueError("gate_cap must be positive")
        self.hidden, self.nh, self.dk, self.dv = int(hidden), int(num_heads), int(key_dim), int(value_dim)
        self.cap, self.eps = float(gate_cap), float(norm_eps)
        self.names = {**self.NAMES, **(names or {})}
        self.graph_safe = True         # entries and their state slots are read from the step's device arrays
        self.w_in = None               # [q | k | v | g] rows: one product of the input
        self.w_gates = None            # [i | f] rows: a product of its own, with a float result
        self.b_i: Optional[torch.Tensor] = None
        self.b_f: Optional[torch.Tensor] = None
        self.w_norm: Optional[torch.Tensor] = None    # float32 [heads * dv]
        self.w_o = None

    def step_planners(self):
        return (WALK_SEGMENTS,)

    def cache_spec(self) -> StateSpec:
        return StateSpec(ops.walk_state_shape(self.nh, self.dk, self.dv, ops.WALK_EXP_GATES), torch.float32)

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        n, qk, vv = self.names, self.nh * self.dk, self.nh * self.dv
        return {
            prefix + n["q"]: ParamSpec((qk, self.hidden)),
            prefix + n["k"]: ParamSpec((qk, self.hidden)),
            prefix + n["v"]: ParamSpec((vv, self.hidden)),
            prefix + n["g"]: ParamSpec((vv, self.hidden)),
            prefix + n["o"]: ParamSpec((self.hidden, vv)),
            prefix + n["norm"]: ParamSpec((vv,), INIT_NORM_WEIGHT),
            prefix + n["i"]: ParamSpec((self.nh, self.hidden)),
            prefix + n["i_bias"]: ParamSpec((self.nh,)),
            prefix + n["f"]: ParamSpec((self.nh, self.hidden)),
            prefix + n["f_bias"]: ParamSpec((self.nh,)),
        }

    def load(self, prefix: str, source: TensorSource) -> None:
        n = self.names
        self.w_in = ops.pack_weight(_fuse([source.get(prefix + n[k]) for k in ("q", "k", "v", "g")], self.hidden))
        self.w_gates = ops.pack_weight(_fuse([source.get(prefix + n[k]) for k in ("i", "f")], self.hidden))
        self.b_i = source.get(prefix + n["i_bias"]).float().contiguous()
        self.b_f = source.get(prefix + n["f_bias"]).float().contiguous()
        self.w_norm = source.get(prefix + n["norm"]).float().contiguous()
        self.w_o = ops.pack_weight(source.get(prefix + n["o"]))

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        if not cache.write:
            raise ValueError("a recurrent mixer's state cannot be shared between layers")
        T = x.shape[0]
        qk, vv = self.nh * self.dk, self.nh * self.dv
        width = 2 if ctx.act_dtype == torch.bfloat16 else 4
        n_in = 2 * qk + 2 * vv
        with section("q|k|v|g", nbytes=width * n_in * (self.hidden + T) + width * T * self.hidden, flops=2.0 * T * self.hidden * n_in):
            proj = ops.linear(x, self.w_in, ctx.act_dtype)
        with section("gates", nbytes=width * 2 * self.nh * self.hidden + width * T * self.hidden + 8 * T * self.nh,
                     flops=4.0 * T * self.hidden * self.nh):
            gates = ops.linear(x, self.w_gates, torch.float32)
        state = cache.states[0] if cache.states else cache.state
        with section("recurrence", nbytes=lambda: 8 * ctx.n_entries * qk * self.dv + T * (width * (2 * qk + vv) + 4 * vv),
                     flops=4.0 * T * qk * self.dv):
            o = ops.state_walk(proj, 0, qk, 2 * qk, 1, gates, (self.b_i, self.b_f), self.cap, self.dk ** -0.5,
                               ops.WALK_EXP_GATES, state, ctx, self.nh, self.dk, self.dv,
                               segments=_segments_for(ctx, self.nh, self.dv))
        with section("head norm + gate", nbytes=T * vv * (4 + 2 * width)):
            y = ops.group_norm_gate(o, self.w_norm, self.eps, self.nh, ctx.act_dtype, proj, 2 * qk + vv, ops.GATE_SIGMOID_ACT)
        with section("o", nbytes=width * self.hidden * (vv + T) + width * T * vv, flops=2.0 * T * self.hidden * vv):
            return ops.linear(y, self.w_o, ctx.act_dtype)


class StateSpaceMixer(Part):
    """A selective state space in its scalar-decay form (Mamba-2).  With h the input, inner = heads * dv,
    N the state's size and G groups: W_in h = [z: inner | x: inner | B: G N | C: G N | dt: heads].  x, B and C
    pass a causal convolution per channel (``conv`` taps, with a bias) and SiLU; dt = softplus(dt + dt_bias).
    Per head (whose group is head // (heads / G)): S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t x_t^T
    (S is N x dv), y_t = S_t^T C_t + D x_t.  The heads side by side are multiplied by silu(z), then
    RMS-normed in ``norm_groups`` equal parts, times a learned weight per channel, then W_o.

    Kept per request, in its state slot: the states S (``ops.walk_state_shape``) and the last
    conv - 1 inputs of the convolution (float).  The step size's product is one of its own with a float
    result; the step sizes, the decays, the state and the norm are float whatever the activations
    are stored as."""

    NAMES = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "A_log": "A_log", "D": "D",
             "norm": "norm", "o": "o"}

    def __init__(self, hidden: int, num_heads: int, value_dim: int, state_dim: int, groups: int, conv_taps: int,
                 norm_groups: int, norm_eps: float, names: Optional[Dict[str, str]] = None):
        if min(num_heads, value_dim, state_dim, groups, norm_groups) < 1 or num_heads % groups or (num_heads * value_dim) % norm_groups:
            raise ValueError("heads, value_dim, state_dim must be positive, groups divide heads, norm_groups divide heads * value_dim")
        if state_dim > ops.WALK_MAX_KEY_DIM:
            raise ValueError(f"a state of {state_dim} elements is not taken: at most {ops.WALK_MAX_KEY_DIM}")
        if not 1 <= conv_taps <= ops.SHORT_CONV_MAX_TAPS:
            raise ValueError(f"a convolution of {conv_taps} taps is not taken: 1 to {ops.SHORT_CONV_MAX_TAPS}")
        self.hidden, self.nh, self.dv, self.N, self.G = int(hidden), int(num_heads), int(value_dim), int(state_dim), int(groups)
        self.taps, self.norm_groups, self.eps = int(conv_taps), int(norm_groups), float(norm_eps)
        self.inner = self.nh * self.dv
        self.conv_channels = self.inner + 2 * self.G * self.N
        self.names = {**self.NAMES, **(names or {})}
        self.graph_safe = True
        self.w_in = None               # [z | x | B | C] rows
        self.w_dt = None               # the step sizes' rows: a product of its own, with a float result
        self.w_conv: Optional[torch.Tensor] = None    # float32 [conv channels, taps]
        self.b_conv: Optional[torch.Tensor] = None
        self.dt_bias: Optional[torch.Tensor] = None
        self.a_log: Optional[torch.Tensor] = None
        self.d_skip: Optional[torch.Tensor] = None
        self.w_norm: Optional[torch.Tensor] = None
        self.w_o = None

    def step_planners(self):
        return (WALK_SEGMENTS,)

    def cache_spec(self):
        walk = StateSpec(ops.walk_state_shape(self.nh, self.N, self.dv, ops.WALK_STATE_SPACE), torch.float32)
        if self.taps == 1:
            return walk
        return MixedSpec(None, (walk, StateSpec((self.taps - 1, self.conv_channels), torch.float32)))

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        n = self.names
        return {
            prefix + n["in"]: ParamSpec((self.inner + self.conv_channels + self.nh, self.hidden)),
            prefix + n["conv"]: ParamSpec((self.conv_channels, self.taps)),
            prefix + n["conv_bias"]: ParamSpec((self.conv_channels,)),
            prefix + n["dt_bias"]: ParamSpec((self.nh,)),
            prefix + n["A_log"]: ParamSpec((self.nh,)),
            prefix + n["D"]: ParamSpec((self.nh,)),
            prefix + n["norm"]: ParamSpec((self.inner,), INIT_NORM_WEIGHT),
            prefix + n["o"]: ParamSpec((self.hidden, self.inner)),
        }

    def load(self, prefix: str, source: TensorSource) -> None:
        n = self.names
        w = source.get(prefix + n["in"])
        split = self.inner + self.conv_channels
        self.w_in = ops.pack_weight(w[:split].contiguous())
        self.w_dt = ops.pack_weight(w[split:].contiguous())
        del w
        self.w_conv = source.get(prefix + n["conv"]).float().contiguous()
        self.b_conv = source.get(prefix + n["conv_bias"]).float().contiguous()
        self.dt_bias = source.get(prefix + n["dt_bias"]).float().contiguous()
        self.a_log = source.get(prefix + n["A_log"]).float().contiguous()
        self.d_skip = source.get(prefix + n["D"]).float().contiguous()
        self.w_norm = source.get(prefix + n["norm"]).float().contiguous()
        self.w_o = ops.pack_weight(source.get(prefix + n["o"]))

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        if not cache.write:
            raise ValueError("a recurrent mixer's state cannot be shared between layers")
        T = x.shape[0]
        width = 2 if ctx.act_dtype == torch.bfloat16 else 4
        n_in = self.inner + self.conv_channels
        with section("z|x|B|C", nbytes=width * n_in * (self.hidden + T) + width * T * self.hidden, flops=2.0 * T * self.hidden * n_in):
            proj = ops.linear(x, self.w_in, ctx.act_dtype)
        with section("gates", nbytes=width * self.nh * self.hidden + width * T * self.hidden + 4 * T * self.nh,
                     flops=2.0 * T * self.hidden * self.nh):
            dt = ops.linear(x, self.w_dt, torch.float32)
        states = cache.states if cache.states else (cache.state,)
        with section("short convolution", nbytes=2 * width * T * self.conv_channels):
            xbc = ops.short_conv(proj, self.inner, self.conv_channels, self.w_conv, self.b_conv,
                                 states[1] if self.taps > 1 else None, ctx)
        with section("recurrence", nbytes=lambda: 8 * ctx.n_entries * self.nh * self.N * self.dv + T * (width * self.conv_channels + 4 * self.inner),
                     flops=4.0 * T * self.nh * self.N * self.dv):
            y = ops.state_walk(xbc, self.inner + self.G * self.N, self.inner, 0, self.nh // self.G, dt,
                               (self.dt_bias, self.a_log, self.d_skip), 0.0, 1.0, ops.WALK_STATE_SPACE, states[0], ctx,
                               self.nh, self.N, self.dv, segments=_segments_for(ctx, self.nh, self.dv))
        with section("head norm + gate", nbytes=T * self.inner * (4 + 2 * width)):
            y = ops.group_norm_gate(y, self.w_norm, self.eps, self.norm_groups, ctx.act_dtype, proj, 0, ops.GATE_SILU, gate_first=True)
        with section("o", nbytes=width * self.hidden * (self.inner + T) + width * T * self.inner, flops=2.0 * T * self.hidden * self.inner):
            return ops.linear(y, self.w_o, ctx.act_dtype)


class Retention(Part):
    """Retention: linear attention with one fixed decay per head, no softmax and no denominator.  With h the
    input, per head (dk key channels, dv value channels): q = W_q h, k = W_k h, v = W_v h; q and k are turned
    by rotary positions (``rotary``: pairs (i, i + r/2) of the leading r elements; None: no rotation), k is then
    multiplied by dk^(-1/2); S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t; each head's output is divided by
    its root mean square (no weight), the heads side by side are multiplied by silu(W_g h) and projected by W_o.

    What is kept per request is S alone, in its state slot (``ops.walk_state_shape``): no pages.  The
    rotation (on the staged floats, inside the walk), the state, its sums and the norm are float whatever
    the activations are stored as.  A step walks each entry's tokens in order from the slot's state
    (csrc/state_walk.hip), long entries in segments side by side."""

    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o"}

    def __init__(self, hidden: int, num_heads: int, key_dim: int, value_dim: int, decays, norm_eps: float, rotary=None,
                 names: Optional[Dict[str, str]] = None):
        if min(num_heads, key_dim, value_dim) < 1:
            raise ValueError("heads, key_dim and value_dim must be positive")
        if key_dim > ops.WALK_MAX_KEY_DIM:
            raise ValueError(f"{key_dim} key channels a head are not taken: at most {ops.WALK_MAX_KEY_DIM}")
        decays = [float(d) for d in decays]
        if len(decays) != num_heads or not all(0.0 < d <= 1.0 for d in decays):
            raise ValueError("one decay in (0, 1] per head is wanted")
        if rotary is not None and (rotary.pair_layout != "half" or rotary.head_dim != key_dim):
            raise ValueError("retention turns split halves of its own key width")
        self.hidden, self.nh, self.dk, self.dv = int(hidden), int(num_heads), int(key_dim), int(value_dim)
        self.decays, self.eps, self.rotary = decays, float(norm_eps), rotary
        self.names = {**self.NAMES, **(names or {})}
        self.graph_safe = True         # entries and their state slots are read from the step's device arrays
        self.w_in = None               # [q | k | v | g] rows: one product of the input
        self.w_o = None
        self._decay_t: Optional[torch.Tensor] = None

    def step_planners(self):
        return (WALK_SEGMENTS,)

    def cache_spec(self) -> StateSpec:
        return StateSpec(ops.walk_state_shape(self.nh, self.dk, self.dv, ops.WALK_FIXED_DECAY), torch.float32)

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        n, qk, vv = self.names, self.nh * self.dk, self.nh * self.dv
        return {
            prefix + n["q"]: ParamSpec((qk, self.hidden)),
            prefix + n["k"]: ParamSpec((qk, self.hidden)),
            prefix + n["v"]: ParamSpec((vv, self.hidden)),
            prefix + n["g"]: ParamSpec((vv, self.hidden)),
            prefix + n["o"]: ParamSpec((self.hidden, vv)),
        }

    def load(self, prefix: str, source: TensorSource) -> None:
        n = self.names
        parts = [source.get(prefix + n[k]) for k in ("q", "k", "v", "g")]
        self.w_in = ops.pack_weight(_fuse(parts, self.hidden))
        self.w_o = ops.pack_weight(source.get(prefix + n["o"]))
        self._decay_t = torch.tensor(self.decays, dtype=torch.float32, device=parts[0].device)

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        if not cache.write:
            raise ValueError("a recurrent mixer's state cannot be shared between layers")
        T = x.shape[0]
        qk, vv = self.nh * self.dk, self.nh * self.dv
        width = 2 if ctx.act_dtype == torch.bfloat16 else 4
        n_in = 2 * qk + 2 * vv
        with section("q|k|v|g", nbytes=width * n_in * (self.hidden + T) + width * T * self.hidden, flops=2.0 * T * self.hidden * n_in):
            proj = ops.linear(x, self.w_in, ctx.act_dtype)
        state = cache.states[0] if cache.states else cache.state
        with section("recurrence", nbytes=lambda: 8 * ctx.n_entries * qk * self.dv + T * (width * (2 * qk + vv) + 4 * vv),
                     flops=4.0 * T * qk * self.dv):
            o = ops.state_walk(proj, 0, qk, 2 * qk, 1, None, (self._decay_t,), 0.0, 1.0, ops.WALK_FIXED_DECAY, state, ctx,
                               self.nh, self.dk, self.dv, segments=_segments_for(ctx, self.nh, self.dv),
                               inv_freq=self.rotary.table(x.device) if self.rotary is not None else None,
                               k_scale=self.dk ** -0.5)
        with section("head norm + gate", nbytes=T * vv * (4 + 2 * width)):
            y = ops.group_norm_gate(o, None, self.eps, self.nh, ctx.act_dtype, proj, 2 * qk + vv, ops.GATE_SILU)
        with section("o", nbytes=width * self.hidden * (vv + T) + width * T * vv, flops=2.0 * T * self.hidden * vv):
            return ops.linear(y, self.w_o, ctx.act_dtype)
