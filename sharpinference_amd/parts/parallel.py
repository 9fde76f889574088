"""Mixers that run side by side on the same input."""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .. import ops
from ..cache.spec import combine_specs, kv_of, states_of
from ..ops.profile import section
from .base import INIT_NORM_WEIGHT, LayerCache, ParamSpec, Part, StepContext, TensorSource


class ParallelMixers(Part):
    """Several mixers read the same input; the result is the mean of their outputs, each first
    RMS-normed over the model width with learned weights of its own:
    y = (1 / n) * sum_b unit_rms(mixer_b(h)) * w_b.

    ``branches``: (name, mixer) pairs; branch b's tensors lie under ``<prefix><name>.`` and its norm
    weight is ``<prefix><name>.<out_name>``.  At most one branch may keep pages; the fixed-size
    states of all of them are asked for together and handed back to each in its own order.  The
    join is float (statistics, weights, the sum); ``forward`` returns it as an ``ops.BranchMean``, which
    the norm kernel behind the mixer forms itself (``tensor()`` forms it for anyone else).

    ``scales`` (one number a branch): the join is instead the plain sum of the outputs with these
    scales, y = sum_b scales[b] * mixer_b(h), without norms or weights of its own; ``forward`` then
    returns an ``ops.BranchSum``, formed in float where it is added to the residual sum."""

    def __init__(self, hidden: int, branches: Sequence[Tuple[str, Part]], norm_eps: float, out_name: str = "out",
                 scales: Optional[Sequence[float]] = None):
        if not 1 <= len(branches) <= ops.NORM_MEAN_MAX_BRANCHES:
            raise ValueError(f"1 to {ops.NORM_MEAN_MAX_BRANCHES} mixers side by side are taken")
        if scales is not None and len(scales) != len(branches):
            raise ValueError("a scale for every branch is wanted")
        self.scales = None if scales is None else [float(s) for s in scales]
        self.hidden, self.eps, self.out_name = int(hidden), float(norm_eps), out_name
        self.branches: List[Tuple[str, Part]] = list(branches)
        self.w_out: List[torch.Tensor] = []
        self.graph_safe = all(getattr(m, "graph_safe", False) or not states_of(self._spec_of(m)) for _, m in self.branches)

    @staticmethod
    def _spec_of(mixer: Part):
        spec = getattr(mixer, "cache_spec", None)
        return spec() if spec else None

    def cache_spec(self):
        return combine_specs([self._spec_of(m) for _, m in self.branches])

    def step_planners(self):
        out = []
        for _, m in self.branches:
            out.extend(getattr(m, "step_planners", tuple)())
        return out

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        specs: Dict[str, ParamSpec] = {}
        for name, m in self.branches:
            specs.update(m.param_specs(f"{prefix}{name}."))
            if self.scales is None:
                specs[f"{prefix}{name}.{self.out_name}"] = ParamSpec((self.hidden,), INIT_NORM_WEIGHT)
        return specs

    def load(self, prefix: str, source: TensorSource) -> None:
        self.w_out = []
        for name, m in self.branches:
            m.load(f"{prefix}{name}.", source)
            if self.scales is None:
                self.w_out.append(source.get(f"{prefix}{name}.{self.out_name}").float().contiguous())

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        outs, at = [], 0
        for _, m in self.branches:
            spec = self._spec_of(m)
            n_states = len(states_of(spec))
            mine = list(cache.states[at:at + n_states])
            at += n_states
            has_pages = kv_of(spec) is not None
            sub = LayerCache(group=cache.group if has_pages else None, k=cache.k if has_pages else None,
                             v=cache.v if has_pages else None, state=mine[0] if mine else None, write=cache.write, states=mine)
            outs.append(m.forward(x, ctx, sub))
        # the join is left to the norm kernel that follows, which forms it while it reads the branches
        if self.scales is not None:
            return ops.BranchSum(outs, self.scales)
        return ops.BranchMean(outs, self.w_out, self.eps)
