"""How a layer's parts are arranged."""
from __future__ import annotations

from typing import Dict

import torch

from .. import ops
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
