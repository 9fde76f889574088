"""How a layer's parts are arranged."""
from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..ops.profile import section
from .base import LayerCache, ParamSpec, Part, ResidualStream, StepContext, TensorSource


class PreNormBlock(Part):
    """h += mixer(norm1(h)); h += ffn(norm2(h))
    (reference: src/SharpInference.Engine/ForwardPass.cs:1557-1561, 1690-1714).

    The additions are folded into the norm that follows them (see ResidualStream), so a block
    leaves its feed-forward output pending for the next block's first norm.  A feed-forward that
    has ``forward_from_stream(stream, norm, ctx)`` is handed the stream and the second norm instead
    of normalised rows (it must leave the stream as the norm would have).  Names of the four
    parts in the weight file are arguments.  ``ffn`` None (with ``norm2`` None): a layer of a mixer
    alone.  ``after``: a part with ``forward_on_stream(stream, ctx)`` that runs at the layer's end on
    the residual sum itself (it adds the pending branch output first); its tensors lie under
    ``names["after"]``."""

    def __init__(self, norm1: Part, mixer: Part, norm2: Part = None, ffn: Part = None, names=None, after: Part = None):
        if (norm2 is None) != (ffn is None):
            raise ValueError("a feed-forward and its norm come together")
        self.norm1, self.mixer, self.norm2, self.ffn, self.after_part = norm1, mixer, norm2, ffn, after
        self.names = dict(names or {"norm1": "input_layernorm.", "mixer": "self_attn.",
                                    "norm2": "post_attention_layernorm.", "ffn": "feed_forward."})

    def _children(self):
        kids = [(self.names["norm1"], self.norm1), (self.names["mixer"], self.mixer)]
        if self.ffn is not None:
            kids += [(self.names["norm2"], self.norm2), (self.names["ffn"], self.ffn)]
        if getattr(self, "after_part", None) is not None:
            kids.append((self.names.get("after", "after."), self.after_part))
        return tuple(kids)

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        out: Dict[str, ParamSpec] = {}
        for name, part in self._children():
            out.update(part.param_specs(prefix + name))
        return out

    def load(self, prefix: str, source: TensorSource) -> None:
        for name, part in self._children():
            part.load(prefix + name, source)

    def step_planners(self):
        out = []
        for _, part in self._children():
            out.extend(getattr(part, "step_planners", tuple)())
        return out

    def cache_spec(self):
        spec = getattr(self.mixer, "cache_spec", None)
        return spec() if spec else None

    def decode_graph_safe(self) -> bool:
        """Can a decode step through this block be captured into a graph?  Paged attention can; a
        mixer with state of its own says so itself (``graph_safe``)."""
        from ..cache.spec import states_of

        return not states_of(self.cache_spec()) or bool(getattr(self.mixer, "graph_safe", False))

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: LayerCache) -> None:
        n = self.norm1.forward(stream, ctx.act_dtype)
        stream.pending = self.mixer.forward(n, ctx, cache)
        from_stream = getattr(self.ffn, "forward_from_stream", None)
        if from_stream is not None:    # a feed-forward that may fuse the norm with work of its own
            stream.pending = from_stream(stream, self.norm2, ctx)
        elif self.ffn is not None:
            n = self.norm2.forward(stream, ctx.act_dtype)
            stream.pending = self.ffn.forward(n, ctx)
        if self.after_part is not None:
            self.after_part.forward_on_stream(stream, ctx)


class PostNormBlock(PreNormBlock):
    """h += norm1(mixer(h)); h += norm2(ffn(h)): the branches read the residual sum itself and the
    norms sit on their outputs.  ``ffn`` None: a layer of a mixer alone.  The sum stays float; a
    branch reads it in the activations' storage type, a copy that the norm kernel leaves beside
    the sum (``stream.act``; the sum itself in float32), so a layer costs no launch for it."""

    def __init__(self, norm1: Part, mixer: Part, norm2: Part = None, ffn: Part = None, names=None):
        if (norm2 is None) != (ffn is None):
            raise ValueError("a feed-forward and its norm come together")
        super().__init__(norm1, mixer, norm2, ffn, names or {"norm1": "norm1.", "mixer": "mixer.", "norm2": "norm2.", "ffn": "ffn."})

    def _children(self):
        kids = [(self.names["norm1"], self.norm1), (self.names["mixer"], self.mixer)]
        if self.ffn is not None:
            kids += [(self.names["norm2"], self.norm2), (self.names["ffn"], self.ffn)]
        return tuple(kids)

    @staticmethod
    def _input(stream: ResidualStream, ctx: StepContext) -> torch.Tensor:
        stream.settle()
        if stream.pending is not None:
            raise ValueError("a block with norms on its outputs cannot follow one that leaves its output pending")
        if stream.act is None or stream.act.dtype != ctx.act_dtype:
            stream.act = stream.h if ctx.act_dtype == torch.float32 else ops.cast(stream.h, ctx.act_dtype)
        return stream.act

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: LayerCache) -> None:
        y = self.mixer.forward(self._input(stream, ctx), ctx, cache)
        self.norm1.add_normed(stream, y, ctx.act_dtype)
        if self.ffn is not None:
            y = self.ffn.forward(stream.act, ctx)
            self.norm2.add_normed(stream, y, ctx.act_dtype)


class SandwichBlock(PreNormBlock):
    """h += norm1b(mixer(norm1(h))); h += norm2b(ffn(norm2(h))): a norm before and a norm after each
    branch.  ``ffn`` None: a layer of a mixer alone.  The norm behind a branch and the norm before
    the next branch are one launch (``RMSNorm.after``); the block's last branch output is left
    waiting behind its norm (``stream.pending_norm``) for the next block's first norm, or for
    whoever settles the stream."""

    def __init__(self, norm1: Part, mixer: Part, norm1b: Part, norm2: Part = None, ffn: Part = None, norm2b: Part = None,
                 names=None):
        if not ((norm2 is None) == (ffn is None) == (norm2b is None)):
            raise ValueError("a feed-forward and its two norms come together")
        super().__init__(norm1, mixer, norm2, ffn, names or {"norm1": "norm1.", "mixer": "mixer.", "norm1b": "norm1b.",
                                                             "norm2": "norm2.", "ffn": "ffn.", "norm2b": "norm2b."})
        self.norm1b, self.norm2b = norm1b, norm2b

    def _children(self):
        kids = [(self.names["norm1"], self.norm1), (self.names["mixer"], self.mixer), (self.names["norm1b"], self.norm1b)]
        if self.ffn is not None:
            kids += [(self.names["norm2"], self.norm2), (self.names["ffn"], self.ffn), (self.names["norm2b"], self.norm2b)]
        return tuple(kids)

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: LayerCache) -> None:
        n = self.norm1.forward(stream, ctx.act_dtype)           # (with the norm behind the branch a block before left waiting)
        y = self.mixer.forward(n, ctx, cache)
        if self.ffn is None:
            stream.pending, stream.pending_norm = y, self.norm1b    # waits for the next norm's launch (or `settle`)
            return
        n = self.norm2.after(self.norm1b, stream, y, ctx.act_dtype)
        stream.pending, stream.pending_norm = self.ffn.forward(n, ctx), self.norm2b


class HyperConnection(Part):
    """The weights by which one sublayer reads S residual streams and writes back into them: ``in`` [S]
    (the sublayer's input is sum_s in[s] x_s), ``mix`` [S, S] indexed (from, to) and ``out`` [S] (every stream
    at once, from the old ones: x_t <- sum_s mix[s, t] x_s + out[t] y).  Kept in float."""

    def __init__(self, n_streams: int, names=None):
        self.S = int(n_streams)
        self.names = dict(names or {"in": "in", "out": "out", "mix": "mix"})
        self.w_in = self.w_out = self.w_mix = None

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        return {prefix + self.names["in"]: ParamSpec((self.S,)), prefix + self.names["out"]: ParamSpec((self.S,)),
                prefix + self.names["mix"]: ParamSpec((self.S, self.S))}

    def load(self, prefix: str, source: TensorSource) -> None:
        self.w_in = source.get(prefix + self.names["in"]).float().contiguous()
        self.w_out = source.get(prefix + self.names["out"]).float().contiguous()
        self.w_mix = source.get(prefix + self.names["mix"]).float().contiguous()


class HyperBlock(PreNormBlock):
    """A pre-norm layer over S residual streams per token instead of one (hyper-connections): for each
    sublayer (the mixer, then the feed-forward where there is one) u = sum_s in[s] x_s, y = sublayer(norm(u)),
    and x_t <- sum_s mix[s, t] x_s + out[t] y for all streams at once.  The streams all start as the embedding
    row, and the model's output reads their plain sum.

    The streams live in ``stream.lanes`` (float32 [T, S, W]); a sublayer's output waits in ``stream.pending``
    with its connection's weights (``stream.pending_lanes``) for the next launch of the one kernel
    (csrc/hyper.hip) that brings the streams up to date, forms the next sublayer's input and normalises
    it; the last output of the model is folded in where the streams are summed (``stream.close()``)."""

    def __init__(self, n_streams: int, norm1: Part, mixer: Part, norm2: Part = None, ffn: Part = None, names=None):
        super().__init__(norm1, mixer, norm2, ffn, names or {"norm1": "norm1", "mixer": "mix.", "norm2": "norm2", "ffn": "mlp.",
                                                             "hc1": "hc1.", "hc2": "hc2."})
        if not 1 <= n_streams <= ops.HYPER_MAX_STREAMS:
            raise ValueError(f"{n_streams} residual streams are not taken: 1 to {ops.HYPER_MAX_STREAMS}")
        self.S = int(n_streams)
        self.hc1 = HyperConnection(self.S)
        self.hc2 = HyperConnection(self.S) if ffn is not None else None

    def _children(self):
        kids = list(super()._children()) + [(self.names["hc1"], self.hc1)]
        if self.hc2 is not None:
            kids.append((self.names["hc2"], self.hc2))
        return tuple(kids)

    def _read(self, stream: ResidualStream, hc: HyperConnection, norm: Part, ctx: StepContext) -> torch.Tensor:
        """The streams brought up to date with the output that waits, and the next sublayer's normalised input."""
        T, W = stream.h.shape
        if stream.lanes is None:
            if stream.pending is not None or stream.pending_norm is not None:
                raise ValueError("a block of several streams cannot follow one that leaves its output pending")
            stream.lanes = torch.empty(T, self.S, W, dtype=torch.float32, device=stream.h.device)
            src = stream.h                                   # every stream starts as this one row
            stream.closer = _sum_of_lanes
        else:
            if stream.lanes.shape[1] != self.S:
                raise ValueError("the layers of a model keep one number of residual streams")
            src = stream.lanes
        delta, mix, out_w = stream.pending, None, None
        if delta is not None:
            mix, out_w = stream.pending_lanes
        with section("norm", nbytes=T * W * (8 * self.S + 4)):
            n = ops.hyper_step(src, stream.lanes, self.S, delta, mix, out_w, hc.w_in, norm.weight, norm.eps, ctx.act_dtype)
        stream.pending = stream.pending_lanes = None
        return n

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: LayerCache) -> None:
        n = self._read(stream, self.hc1, self.norm1, ctx)
        stream.pending, stream.pending_lanes = self.mixer.forward(n, ctx, cache), (self.hc1.w_mix, self.hc1.w_out)
        if self.ffn is not None:
            n = self._read(stream, self.hc2, self.norm2, ctx)
            stream.pending, stream.pending_lanes = self.ffn.forward(n, ctx), (self.hc2.w_mix, self.hc2.w_out)


def _sum_of_lanes(stream: ResidualStream, rows) -> bool:
    """h = the plain sum of the streams, the waiting output folded in first, for the rows asked for
    alone (the streams themselves are not stored again: nobody reads them after this)."""
    S = stream.lanes.shape[1]
    delta, mix, out_w = stream.pending, None, None
    if delta is not None:
        mix, out_w = stream.pending_lanes
    n = stream.h.shape[0] if rows is None else rows.shape[0]
    with section("norm", nbytes=n * stream.h.shape[1] * (4 * S + 4)):
        stream.h = ops.hyper_step(stream.lanes, None, S, delta, mix, out_w, rows=rows)
    stream.pending = stream.pending_lanes = stream.lanes = None
    return rows is not None
