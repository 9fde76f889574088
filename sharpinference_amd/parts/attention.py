"""The attention mixer: grouped-query attention over the paged cache."""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

from .. import ops
from ..ops.lib import PREFILL_TILE_TOKENS
from ..ops.profile import section
from ..cache.spec import KVSpec, MixedSpec, StateSpec, kv_of, WINDOW_CHUNK, WINDOW_NONE, WINDOW_SLIDING  # noqa: F401
from .base import INIT_NORM_WEIGHT, HostStep, LayerCache, ParamSpec, Part, StepContext, StepPlanner, TensorSource

SHORT_PROMPT_TOKENS = 1536   # up to so many prompt tokens in a step, tiles of half as many tokens (measured:
                             # 20-25 % less attention time from 512 to 1,536 tokens, 6 % more at 2,048)


class AttentionWorkLists(StepPlanner):
    """How the attention kernels split a batch: the tokens of entries of one token (the split-K
    decode kernel's list; none when every token is one, the kernel then takes them all) and the
    tiles of the longer entries (entry, first token, rows) for the flash kernel.  A step with few
    prompt tokens is cut into tiles of half the rows: its attention launch lasts as long as its
    longest tile, and twice the blocks of half the rows walk their keys faster."""

    key = "attention"

    def plan(self, host: HostStep) -> Tuple[List[np.ndarray], dict]:
        lens, cu = host.lens, host.cu_tokens
        dec = [int(cu[i]) for i in range(host.n_entries) if lens[i] == 1]
        tile = PREFILL_TILE_TOKENS if sum(n for n in lens if n > 1) > SHORT_PROMPT_TOKENS else PREFILL_TILE_TOKENS // 2
        tiles = [(i, int(cu[i]) + o, min(tile, lens[i] - o)) for i in range(host.n_entries) if lens[i] > 1
                 for o in range(0, lens[i], tile)]
        arrays = [np.asarray(dec, dtype=np.int32), np.asarray(tiles, dtype=np.int32).reshape(-1)]
        return arrays, dict(n_dec=len(dec), n_tiles=len(tiles), tile=tile, all_decode=len(dec) == host.n_tokens)

    def null(self, host: HostStep, arrays: List[np.ndarray]) -> List[np.ndarray]:
        return [np.arange(arrays[0].size, dtype=np.int32), np.zeros_like(arrays[1])]

    def attach(self, ctx: StepContext, views: List[torch.Tensor], facts: dict) -> None:
        ctx.n_decode = facts["n_dec"]
        ctx.decode_tokens = None if facts["all_decode"] else views[0]
        ctx.n_prefill_tiles = facts["n_tiles"]
        ctx.prefill_tiles = views[1].view(-1, 3) if facts["n_tiles"] else None
        ctx.prefill_tile_tokens = facts["tile"]


_WORK_LISTS = AttentionWorkLists()


class Attention(Part):
    """q/k/v projections (with biases if ``bias``) -> position encoding -> optional weightless per-head norm
    -> optional query temperature -> keys and values into the cache -> softmax(q k^T * scale) v
    over the keys the window admits -> output projection
    (reference: src/SharpInference.Engine/ForwardPass.cs:1576-1690, 1838-1912; the norm comes
    after the rotation, 1643-1648; optional biases are added right after their products,
    1605-1613, the output projection's may be absent on its own, 381-383).

    Everything that differs between layers is an argument: ``rotary`` (None = no position
    encoding; otherwise any object with ``table(device)``, ``pair_layout``, ``rotary_dim`` and
    ``head_dim``, see parts/position.py), ``v_head_dim`` (values and a head's output of another width than
    keys: such layers run the float attention kernel), ``qk_norm_eps`` (None = no norm), ``q_temperature`` = (floor_scale, attn_scale)
    multiplying queries by 1 + attn_scale * ln(floor((pos + 1) / floor_scale) + 1), and the
    window: all keys, the chunk [floor(pos/W)*W, pos], or the last W keys.

    Further options, for designs that norm before they rotate (they take the other kernel between
    the projections and attention, csrc/qk_prep.hip):
    ``qk_norm_weights``: "head" (an RMS norm of every query and key head with learned weights [head_dim]
    shared by the heads) or "projection" (one RMS norm over all of a token's query heads, and one
    over all its key heads, weights [heads * head_dim]); eps is ``qk_norm_eps``; the norm comes
    BEFORE the rotation.  ``values_from_keys``: no value projection; a value is its key as
    projected, before norm and rotation.  ``conv_taps`` n >= 2: a causal convolution over time on
    every channel of q, k and v right behind the projections, y_t = sum_j w[:, j] u_(t - n + 1 + j)
    (weights [channels, n]; zeros before a sequence's start; the last n - 1 projected rows of a
    request are carried in its state slot).  ``softcap`` c: scores become c tanh(score / c).
    ``sink``: the softmax's denominator holds one more term exp(0), a key of score 0 that has no
    value; ``sink="learned"``: the term is exp(s_h) with a stored number s_h per head (tensor
    ``sink`` [heads], float; not scaled).  ``gate``: the heads' outputs side by side are multiplied
    element by element by sigmoid(W_g x) (W_g [heads * v_head_dim, hidden], a product of the same
    input as q, k and v, made by the same launch) before the output projection.  A rotary object's
    ``magnitude`` multiplies cos and sin.  ``names``: the tensors' names behind the layer's prefix.

    ``score_maps`` m > 1 with ``difference`` c: differential attention.  Every query head and every key head
    holds m = 2 score maps of ``head_dim`` elements side by side (q rows [head][map][head_dim], and so k); each
    map is an attention of its own (position encoding per map, the same scale, window and softmax) over the
    head's one set of values, and the head's output is unit_rms(a_1 - lambda a_2) * (1 - c) with
    lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + c from four stored vectors [head_dim], one number for the
    layer, the root mean square over the head's values with ``difference_eps`` inside the root.  The cache
    keeps a key head's maps as one row of m * head_dim elements; queries are expanded to one such row per
    (head, map) with zeros in the other map's place, so the attention kernels compute each map's scores
    unchanged (csrc/qk_prep.hip, csrc/hyper.hip).  ``head_gate``: each head's output is multiplied by
    sigmoid(W_g x)_h, one number per head (W_g [heads, hidden], made by the q|k|v launch)."""

    NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
             "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias", "o_bias": "o_proj.bias",
             "q_norm": "q_norm.weight", "k_norm": "k_norm.weight",
             "q_conv": "q_conv.weight", "k_conv": "k_conv.weight", "v_conv": "v_conv.weight",
             "sink": "sink", "g": "g_proj.weight", "lq1": "lq1", "lk1": "lk1", "lq2": "lq2", "lk2": "lk2"}

    def __init__(self, hidden: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 rotary=None, qk_norm_eps: Optional[float] = None,
                 q_temperature: Optional[Tuple[float, float]] = None, window_kind: int = WINDOW_NONE,
                 window: int = 0, scale: Optional[float] = None, bias: bool = False, o_bias: Optional[bool] = None,
                 v_head_dim: Optional[int] = None, qk_norm_weights: Optional[str] = None, values_from_keys: bool = False,
                 conv_taps: int = 0, softcap: float = 0.0, sink=False, names: Optional[Dict[str, str]] = None,
                 gate: bool = False, score_maps: int = 1, difference: Optional[float] = None,
                 difference_eps: Optional[float] = None, head_gate: bool = False):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads cannot share {num_kv_heads} kv heads")
        self.maps = int(score_maps)
        if self.maps not in (1, 2) or (self.maps == 2) != (difference is not None):
            raise ValueError("score_maps is 1, or 2 together with the difference's constant")
        if self.maps == 2 and (difference_eps is None or not 0.0 <= float(difference) < 1.0):
            raise ValueError("differential attention needs difference_eps and a constant in [0, 1)")
        self.difference = float(difference) if difference is not None else 0.0
        self.difference_eps = float(difference_eps) if difference_eps is not None else 0.0
        self.head_gate = bool(head_gate)
        if self.head_gate and (gate or self.maps == 1):
            raise ValueError("a gate number per head belongs to differential attention and excludes the gate per channel")
        prep = bool(qk_norm_weights or values_from_keys or conv_taps or self.maps > 1)
        self.map_dim = int(head_dim)                      # width of one score map of a head
        if rotary is not None and rotary.head_dim != head_dim:
            raise ValueError("the rotary table's head_dim differs from the mixer's")
        head_dim = int(head_dim) * self.maps              # a head as the cache and the kernels see it: its maps side by side
        widest = 256 * self.maps                          # (the rotation takes pairs; the attention kernels hold 256 elements a map)
        if head_dim % 2 or not 2 <= head_dim <= widest:
            raise ValueError(f"head_dim {head_dim} is not taken: even sizes from 2 to {widest}")
        if rotary is not None and rotary.pair_layout not in ("interleaved", "half"):
            raise ValueError(f"pair layout {rotary.pair_layout!r} is not taken by the rotation kernel")
        self.hidden, self.nh, self.nkv, self.hd = int(hidden), int(num_heads), int(num_kv_heads), int(head_dim)
        self.vd = int(v_head_dim or head_dim)                    # width of a value (and of a head's output)
        if not 1 <= self.vd <= 256:
            raise ValueError(f"v_head_dim {self.vd} is not taken: 1 to 256")
        self.rotary, self.qk_norm_eps, self.q_temperature = rotary, qk_norm_eps, q_temperature
        self.window_kind, self.window = int(window_kind), int(window)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.bias = bool(bias)                                   # q, k and v carry biases
        self.o_bias = self.bias if o_bias is None else bool(o_bias)   # the output projection carries one
        if qk_norm_weights not in (None, "head", "projection"):
            raise ValueError(f"qk_norm_weights {qk_norm_weights!r} is not known (None, 'head', 'projection')")
        if qk_norm_weights and qk_norm_eps is None:
            raise ValueError("a norm with weights needs qk_norm_eps")
        if values_from_keys and self.vd != self.hd:
            raise ValueError("values taken from the keys have the keys' width")
        self.conv_taps = int(conv_taps)
        if self.conv_taps and not 2 <= self.conv_taps <= ops.QK_PREP_MAX_TAPS:
            raise ValueError(f"a convolution of {conv_taps} taps is not taken: 2 to {ops.QK_PREP_MAX_TAPS}")
        self.qk_norm_weights, self.values_from_keys = qk_norm_weights, bool(values_from_keys)
        if sink not in (False, True, None, "learned"):
            raise ValueError(f"sink {sink!r} is not known (False, True, 'learned')")
        self.softcap, self.sink = float(softcap or 0.0), bool(sink)
        self.learned_sink, self.has_gate = sink == "learned", bool(gate)
        if self.has_gate and prep:
            raise ValueError("an output gate belongs to the rotate-then-norm form of the layer")
        if self.softcap < 0:
            raise ValueError("softcap must be positive (or 0 for none)")
        if self.maps > 1 and (self.sink or self.softcap):
            raise ValueError("differential attention comes without a sink and without a cap on the scores")
        self.prep = prep                                         # the layer takes the norm-before-rotation kernel
        if prep and bias and conv_taps:
            raise ValueError("q/k/v biases and a convolution behind the projections do not come together")
        if prep and self.o_bias:
            raise ValueError("an output bias belongs to the rotate-then-norm form of the layer")
        if prep and (self.nh + 2 * self.nkv) * max(self.hd, self.vd) > ops.QK_PREP_MAX_ROW:
            raise ValueError(f"a token's q, k and v of more than {ops.QK_PREP_MAX_ROW} channels are not taken")
        if not prep and rotary is not None and getattr(rotary, "magnitude", 1.0) != 1.0:
            raise ValueError("a rotation with a magnitude belongs to the norm-before-rotation form of the layer")
        self.graph_safe = True                                   # its state (a convolution's tail) is walked on the device
        self.names = {**self.NAMES, **(names or {})}
        self.w_qkv: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None
        self.b_qkv: Optional[torch.Tensor] = None                # float32 [q + 2 kv]: added by the rotation kernel
        self.b_o: Optional[torch.Tensor] = None                  # float32 [hidden]
        self.w_q_norm: Optional[torch.Tensor] = None             # float32
        self.w_k_norm: Optional[torch.Tensor] = None
        self.w_conv: Optional[torch.Tensor] = None               # float32 [q + k + v channels, taps]
        self.w_sink: Optional[torch.Tensor] = None               # float32 [heads]
        self.lam: float = 0.0                                    # the difference's lambda (from four stored vectors)

    # -- what it needs --------------------------------------------------------
    def step_planners(self):
        return (_WORK_LISTS,)

    @property
    def _channels(self) -> int:
        """Projected channels of a token: q, k and (where the layer has a value projection) v."""
        return self.nh * self.hd + self.nkv * self.hd + (0 if self.values_from_keys else self.nkv * self.vd)

    def cache_spec(self):
        kv = KVSpec(self.nkv, self.hd, self.window_kind, self.window, 0 if self.vd == self.hd else self.vd)
        if not self.conv_taps:
            return kv
        return MixedSpec(kv, (StateSpec((self.conv_taps - 1, self._channels), torch.float32),))

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        q, kv, vv, ov = self.nh * self.hd, self.nkv * self.hd, self.nkv * self.vd, self.nh * self.vd
        n = self.names
        specs = {
            prefix + n["q"]: ParamSpec((q, self.hidden)),
            prefix + n["k"]: ParamSpec((kv, self.hidden)),
            prefix + n["o"]: ParamSpec((self.hidden, ov)),
        }
        if not self.values_from_keys:
            specs[prefix + n["v"]] = ParamSpec((vv, self.hidden))
        if self.bias:
            specs.update({prefix + n["q_bias"]: ParamSpec((q,)), prefix + n["k_bias"]: ParamSpec((kv,)),
                          prefix + n["v_bias"]: ParamSpec((vv,))})
        if self.o_bias:
            specs[prefix + n["o_bias"]] = ParamSpec((self.hidden,))
        if self.qk_norm_weights:
            whole = self.qk_norm_weights == "projection"
            specs[prefix + n["q_norm"]] = ParamSpec((q if whole else self.hd,), INIT_NORM_WEIGHT)
            specs[prefix + n["k_norm"]] = ParamSpec((kv if whole else self.hd,), INIT_NORM_WEIGHT)
        if self.learned_sink:
            specs[prefix + n["sink"]] = ParamSpec((self.nh,))
        if self.has_gate:
            specs[prefix + n["g"]] = ParamSpec((ov, self.hidden))
        if self.head_gate:
            specs[prefix + n["g"]] = ParamSpec((self.nh, self.hidden))
        if self.maps > 1:
            for key in ("lq1", "lk1", "lq2", "lk2"):
                specs[prefix + n[key]] = ParamSpec((self.map_dim,))
        if self.conv_taps:
            specs[prefix + n["q_conv"]] = ParamSpec((q, self.conv_taps))
            specs[prefix + n["k_conv"]] = ParamSpec((kv, self.conv_taps))
            if not self.values_from_keys:
                specs[prefix + n["v_conv"]] = ParamSpec((vv, self.conv_taps))
        return specs

    def load(self, prefix: str, source: TensorSource) -> None:
        n = self.names
        kinds = ("q", "k") if self.values_from_keys else ("q", "k", "v")
        parts = [source.get(prefix + n[k]) for k in kinds + (("g",) if self.has_gate or self.head_gate else ())]
        dt = torch.float32 if any(p.dtype == torch.float32 for p in parts) else parts[0].dtype
        fused = torch.empty(sum(p.shape[0] for p in parts), self.hidden, dtype=dt, device=parts[0].device)
        o = 0
        for p in parts:
            fused[o:o + p.shape[0]].copy_(p)
            o += p.shape[0]
        # both also in the order the few-rows kernel streams them; the rows stay for prompt-sized steps
        self.w_qkv = ops.pack_weight(fused)
        self.w_o = ops.pack_weight(source.get(prefix + n["o"]))
        if self.bias:
            self.b_qkv = torch.cat([source.get(prefix + n[k + "_bias"]).float() for k in ("q", "k", "v")]).contiguous()
        if self.o_bias:
            self.b_o = source.get(prefix + n["o_bias"]).float().contiguous()
        if self.qk_norm_weights:
            self.w_q_norm = source.get(prefix + n["q_norm"]).float().contiguous()
            self.w_k_norm = source.get(prefix + n["k_norm"]).float().contiguous()
        if self.learned_sink:
            self.w_sink = source.get(prefix + n["sink"]).float().contiguous()
        if self.maps > 1:
            lq1, lk1, lq2, lk2 = (source.get(prefix + n[key]).float() for key in ("lq1", "lk1", "lq2", "lk2"))
            self.lam = float(torch.exp((lq1 * lk1).sum()) - torch.exp((lq2 * lk2).sum()) + self.difference)
        if self.conv_taps:
            self.w_conv = torch.cat([source.get(prefix + n[k + "_conv"]).float() for k in kinds]).contiguous()

    # -- compute --------------------------------------------------------------
    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        g = cache.group
        T = x.shape[0]
        width = 2 if ctx.act_dtype == torch.bfloat16 else 4
        q_dim, kv_dim = self.nh * self.hd, self.nkv * (self.hd + self.vd) // 2    # (kv_dim: the mean of a key's and a value's row)
        g_dim = self.nh * self.vd if self.has_gate else self.nh if self.head_gate else 0
        with section("qkv", nbytes=width * (q_dim + 2 * kv_dim + g_dim) * (self.hidden + T) + width * T * self.hidden,
                     flops=2.0 * T * self.hidden * (q_dim + 2 * kv_dim + g_dim)):
            qkv = ops.linear(x, self.w_qkv, ctx.act_dtype)
        slots = g.slot_mapping if cache.write else ctx.no_store_slots
        inv_freq = self.rotary.table(x.device) if self.rotary is not None else None
        layout = ops.PAIRS_HALF_SPLIT if self.rotary is not None and self.rotary.pair_layout == "half" else ops.PAIRS_INTERLEAVED
        with section("rope + cache write", nbytes=2 * width * T * (q_dim + 2 * kv_dim)):
            if self.prep:
                mode = {None: ops.NORM_NONE, "head": ops.NORM_PER_HEAD, "projection": ops.NORM_WHOLE}[self.qk_norm_weights]
                kn = self.nkv * self.hd
                q = ops.qk_prep(qkv, 0, q_dim, None if self.values_from_keys else q_dim + kn, self.nh, self.nkv, self.hd,
                                self.vd, ctx, cache.k, cache.v, slots, mode, self.w_q_norm, self.w_k_norm,
                                self.qk_norm_eps or 1e-6, inv_freq, layout,
                                getattr(self.rotary, "magnitude", 1.0) if self.rotary is not None else 1.0,
                                self.w_conv, cache.states[0] if self.conv_taps else None, update_tail=cache.write,
                                bias=self.b_qkv, temperature=self.q_temperature, maps=self.maps)
            else:
                q = ops.rope_kv(qkv, cache.k, cache.v, slots, ctx.positions, inv_freq, self.qk_norm_eps is not None,
                                self.qk_norm_eps or 1e-6, self.q_temperature, self.nh, self.nkv, self.hd, layout,
                                bias=self.b_qkv, vd=self.vd, extra_columns=g_dim)
        with section("attention", nbytes=lambda: self._keys_held(ctx) * 2 * kv_dim * width + 2 * T * q_dim * width,
                     flops=lambda: 4.0 * self._keys_read(ctx) * q_dim):
            o = ops.attention(q, cache.k, cache.v, g, ctx, self.window_kind, self.window, self.scale, self.nh * self.maps,
                              self.nkv, self.hd, self.vd, softcap=self.softcap, sink=self.w_sink if self.learned_sink else self.sink)
        if self.maps > 1:
            with section("difference of the maps", nbytes=3 * width * T * self.nh * self.vd):
                o = ops.map_difference(o, self.nh, self.vd, self.lam, self.difference_eps, 1.0 - self.difference,
                                       qkv if self.head_gate else None, qkv.shape[1] - g_dim)
        if self.has_gate:
            with section("output gate", nbytes=3 * width * T * g_dim):
                o = ops.sigmoid_gate(o, qkv, qkv.shape[1] - g_dim)
        with section("o", nbytes=width * self.hidden * (q_dim + T) + width * T * q_dim, flops=2.0 * T * self.hidden * q_dim):
            out = ops.linear(o, self.w_o, ctx.act_dtype)
            return ops.add_bias(out, self.b_o) if self.b_o is not None else out

    def _keys_read(self, ctx: StepContext) -> int:
        """(query, key) pairs of the step: what is computed."""
        spec = kv_of(self.cache_spec())
        return sum(p - spec.first_visible(p) + 1 for s, n in zip(ctx.entry_starts, ctx.entry_lens) for p in range(s, s + n))

    def _keys_held(self, ctx: StepContext) -> int:
        """Keys that some query of the step sees, each counted once per entry: what has to be read."""
        spec = kv_of(self.cache_spec())
        return sum(s + n - spec.first_visible(s) for s, n in zip(ctx.entry_starts, ctx.entry_lens))
