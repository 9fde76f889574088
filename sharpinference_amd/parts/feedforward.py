"""Feed-forward parts: the dense SwiGLU and the routed mixture of SwiGLU experts."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..ops.profile import active as profiling, section
from .base import ParamSpec, Part, ResidualStream, StepContext, TensorSource
from .norm import RMSNorm


def _fuse_rows(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """[.., Ia, H] and [.., Ib, H] -> [.., Ia + Ib, H] (gate rows first, up rows second)."""
    dt = torch.float32 if torch.float32 in (a.dtype, b.dtype) else a.dtype
    shape = list(a.shape)
    shape[-2] = a.shape[-2] + b.shape[-2]
    out = torch.empty(shape, dtype=dt, device=a.device)
    out[..., : a.shape[-2], :].copy_(a)
    out[..., a.shape[-2]:, :].copy_(b)
    return out


def _rows(w) -> torch.Tensor:
    return ops.unpack_weight(w) if isinstance(w, ops.PackedWeight) else w


def _activation_code(name: str, limit: Optional[float] = None):
    """What the kernels take for the gated unit `name` (a code, or a code with its limit)."""
    if name not in ops.ACTIVATIONS:
        raise ValueError(f"activation {name!r} is not known ({', '.join(sorted(ops.ACTIVATIONS))})")
    return ops.gated_activation(name, limit)


class DenseSwiGLU(Part):
    """down( act(gate x) * (up x) ) (reference: src/SharpInference.Engine/ForwardPass.cs:2006-2015;
    silu(g) = g / (1 + exp(-g)), src/SharpInference.Cpu/SimdKernels.cs:4377-4408).  ``activation``
    names the gate's function: "silu" (the reference's), "gelu_tanh", or "swish_clamp" with ``limit``:
    g = min(gate x, limit), u = clamp(up x, -limit, limit), and the unit is g sigmoid(1.702 g) (u + 1).  ``bias``: the three
    products carry biases (``names`` + ``bias_suffix``), added in float: the gate's and the up
    projection's inside the activation kernel, the down projection's by a row kernel.  ``names``:
    the three matrices' names behind the part's prefix."""

    NAMES = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}

    def __init__(self, hidden: int, intermediate: int, activation: str = "silu", bias: bool = False,
                 names: Optional[Dict[str, str]] = None, bias_suffix: str = ".bias", limit: Optional[float] = None):
        self.hidden, self.inter = int(hidden), int(intermediate)
        self.act = _activation_code(activation, limit)
        self.bias, self.bias_suffix = bool(bias), bias_suffix
        self.names = {**self.NAMES, **(names or {})}
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None
        self.b_gate_up: Optional[torch.Tensor] = None     # float32 [2 * inter]
        self.b_down: Optional[torch.Tensor] = None        # float32 [hidden]

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        n = self.names
        out = {
            prefix + n["gate"]: ParamSpec((self.inter, self.hidden)),
            prefix + n["up"]: ParamSpec((self.inter, self.hidden)),
            prefix + n["down"]: ParamSpec((self.hidden, self.inter)),
        }
        if self.bias:
            out.update({prefix + n["gate"] + self.bias_suffix: ParamSpec((self.inter,)),
                        prefix + n["up"] + self.bias_suffix: ParamSpec((self.inter,)),
                        prefix + n["down"] + self.bias_suffix: ParamSpec((self.hidden,))})
        return out

    def load(self, prefix: str, source: TensorSource) -> None:
        n = self.names
        g = source.get(prefix + n["gate"])
        u = source.get(prefix + n["up"])
        # both also in the order the few-rows kernel streams them; the rows stay for prompt-sized steps
        self.w_gate_up = ops.pack_weight(_fuse_rows(g, u))
        del g, u
        self.w_down = ops.pack_weight(source.get(prefix + n["down"]))
        if self.bias:
            self.b_gate_up = torch.cat([source.get(prefix + n[k] + self.bias_suffix).float() for k in ("gate", "up")]).contiguous()
            self.b_down = source.get(prefix + n["down"] + self.bias_suffix).float().contiguous()

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        T = x.shape[0]
        width = 2 if ctx.act_dtype == torch.bfloat16 else 4
        with section("dense feed-forward", nbytes=width * 3 * self.inter * self.hidden + width * T * (2 * self.hidden + 3 * self.inter),
                     flops=6.0 * T * self.inter * self.hidden):
            gu = ops.linear(x, self.w_gate_up, ctx.act_dtype)
            act = ops.gated_act(gu, None, self.act, bias=self.b_gate_up)
            out = ops.linear(act, self.w_down, ctx.act_dtype)
            return ops.add_bias(out, self.b_down) if self.b_down is not None else out


class DenseMLP(Part):
    """down( act(up x) ): a feed-forward without a gate.  ``activation``: "relu2" (the square of
    relu), "gelu_tanh" or "silu".  ``names``: the two matrices' names behind the part's prefix."""

    def __init__(self, hidden: int, intermediate: int, activation: str = "relu2", names: Optional[Dict[str, str]] = None):
        if activation not in ops.UNGATED_ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not known ({', '.join(sorted(ops.UNGATED_ACTIVATIONS))})")
        self.hidden, self.inter, self.activation = int(hidden), int(intermediate), activation
        self.names = {"up": "up_proj.weight", "down": "down_proj.weight", **(names or {})}
        self.w_up = None
        self.w_down = None

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        return {prefix + self.names["up"]: ParamSpec((self.inter, self.hidden)),
                prefix + self.names["down"]: ParamSpec((self.hidden, self.inter))}

    def load(self, prefix: str, source: TensorSource) -> None:
        self.w_up = ops.pack_weight(source.get(prefix + self.names["up"]))
        self.w_down = ops.pack_weight(source.get(prefix + self.names["down"]))

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        T = x.shape[0]
        width = 2 if ctx.act_dtype == torch.bfloat16 else 4
        with section("dense feed-forward", nbytes=width * 2 * self.inter * self.hidden + width * T * (2 * self.hidden + 3 * self.inter),
                     flops=4.0 * T * self.inter * self.hidden):
            up = ops.linear(x, self.w_up, ctx.act_dtype)
            return ops.linear(ops.activation(up, self.activation), self.w_down, ctx.act_dtype)


class MoESwiGLU(Part):
    """Router -> top-k experts (+ an always-on shared expert)
    (reference: src/SharpInference.Engine/ForwardPass.cs:2021-2098).

    The router's logits, gate and picks are float and stay on the device.  With
    ``score_on_input`` the gate and up products of a chosen expert are multiplied by its score
    before the SiLU (ForwardPass.cs:2083-2089); without it the expert runs on the unscaled input
    and its output is multiplied by the score where the outputs are summed (the reference's other
    order, src/SharpInference.Cuda/CudaKernels.cs:112-157 llm_moe_weighted_reduce).  The shared
    expert sees the unscaled input (2060-2066); the outputs are summed (2096-2097).  ``gate`` is "sigmoid" or "softmax"
    (2031-2034); ``renormalise`` divides the k scores by their sum (2156-2162); ``activation`` names the
    experts' gate function ("silu", the reference's, "gelu_tanh", or "swish_clamp" with ``limit``; the
    shared expert may have a limit and a width of its own, ``shared_limit``).  ``gate`` "softmax_picked":
    the largest logits are picked and their weights are the softmax over the picked logits alone.
    ``router_bias``: a stored vector [E] is added to the router's logits."""

    MERGE_MAX_TOKENS = 16   # one row block of the few-rows kernel for the shared group (measured: up to 64 tokens
                            # the merged launches and the library's product for the shared expert are as fast)
    MERGE_MIN_MANY_TOKENS = None   # tokens from which the shared expert is one more group of the many-rows grouped
                                   # product; off: measured at 2,048 tokens, 1.48 ms a layer against 0.93 + 0.45 with
                                   # the library's product for the shared expert (which runs at the matrix cores' peak)

    NAMES = {"router": "router.weight", "gate": "experts.gate_proj", "up": "experts.up_proj",
             "down": "experts.down_proj", "shared": "shared_expert.", "correction": "router.correction",
             "router_bias": "router.bias"}

    def __init__(self, hidden: int, num_experts: int, top_k: int, expert_intermediate: int,
                 shared_intermediate: Optional[int] = None, gate: str = "sigmoid", renormalise: bool = False,
                 score_on_input: bool = True, activation: str = "silu", correction: bool = False,
                 n_groups: int = 1, keep_groups: int = 1, names: Optional[Dict[str, str]] = None,
                 limit: Optional[float] = None, shared_limit: Optional[float] = None, router_bias: bool = False):
        """``correction``: a stored vector [E] is added to the gate values where experts are chosen
        (the weights stay the gate values).  ``n_groups`` / ``keep_groups``: the experts form
        n_groups equal groups of neighbours and are chosen from the keep_groups best of them only
        (a group's rank: the sum of its two largest choice scores).  ``names``: the tensors' names
        behind the part's prefix; a gate / up / down name with ``{e}`` in it is one matrix per
        expert (stacked when loaded) instead of one stacked tensor."""
        self.names = {**self.NAMES, **(names or {})}
        self.correction = bool(correction)
        self.n_groups, self.keep_groups = int(n_groups), int(keep_groups)
        if not (1 <= self.keep_groups <= self.n_groups and num_experts % self.n_groups == 0
                and top_k <= self.keep_groups * (num_experts // self.n_groups)):
            raise ValueError(f"{n_groups} groups of which {keep_groups} are kept do not fit {num_experts} experts and {top_k} picks")
        self.w_correction: Optional[torch.Tensor] = None
        if not 1 <= top_k <= num_experts:
            raise ValueError(f"top_k {top_k} must lie in 1..{num_experts}")
        if num_experts > ops.ROUTER_MAX_EXPERTS:
            raise ValueError(f"{num_experts} experts are not taken: the routing kernels hold scores for {ops.ROUTER_MAX_EXPERTS}")
        if gate not in ("sigmoid", "softmax", "softmax_picked"):
            raise ValueError(f"router gate {gate!r} is not known (sigmoid, softmax, softmax_picked)")
        self.hidden, self.E, self.k = int(hidden), int(num_experts), int(top_k)
        self.inter = int(expert_intermediate)
        self.act = _activation_code(activation, limit)
        shared_names = {k: self.names[k] for k in ("shared_gate", "shared_up", "shared_down") if k in self.names}
        self.shared = DenseSwiGLU(hidden, shared_intermediate, activation, limit=shared_limit if shared_limit is not None else limit,
                                  names={k[len("shared_"):]: v for k, v in shared_names.items()} or None) if shared_intermediate else None
        self.gate = {"sigmoid": ops.GATE_SIGMOID, "softmax": ops.GATE_SOFTMAX, "softmax_picked": ops.GATE_SOFTMAX_PICKED}[gate]
        self.router_bias = bool(router_bias)
        self.b_router: Optional[torch.Tensor] = None      # float32 [E]
        self.renormalise = bool(renormalise)
        self.score_on_input = bool(score_on_input)
        self.w_router: Optional[torch.Tensor] = None
        self.w_gate_up: Optional[torch.Tensor] = None     # [E, 2*I, H]
        self.w_down: Optional[torch.Tensor] = None        # [E, H, I]

    def _expert_specs(self, prefix: str, which: str, shape) -> Dict[str, ParamSpec]:
        name = self.names[which]
        if "{e}" in name:
            return {prefix + name.format(e=e): ParamSpec(tuple(shape)) for e in range(self.E)}
        return {prefix + name: ParamSpec((self.E, *shape))}

    def _expert_stack(self, prefix: str, which: str, source: TensorSource) -> torch.Tensor:
        name = self.names[which]
        if "{e}" not in name:
            return source.get(prefix + name)
        first = source.get(prefix + name.format(e=0))
        out = torch.empty((self.E, *first.shape), dtype=first.dtype, device=first.device)
        out[0].copy_(first)
        for e in range(1, self.E):
            out[e].copy_(source.get(prefix + name.format(e=e)))
        return out

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        out = {prefix + self.names["router"]: ParamSpec((self.E, self.hidden))}
        out.update(self._expert_specs(prefix, "gate", (self.inter, self.hidden)))
        out.update(self._expert_specs(prefix, "up", (self.inter, self.hidden)))
        out.update(self._expert_specs(prefix, "down", (self.hidden, self.inter)))
        if self.correction:
            out[prefix + self.names["correction"]] = ParamSpec((self.E,))
        if self.router_bias:
            out[prefix + self.names["router_bias"]] = ParamSpec((self.E,))
        if self.shared is not None:
            out.update(self.shared.param_specs(prefix + self.names["shared"]))
        return out

    def _route_args(self) -> dict:
        return dict(correction=self.w_correction, n_groups=self.n_groups, keep_groups=self.keep_groups, bias=self.b_router)

    def load(self, prefix: str, source: TensorSource) -> None:
        self.w_router = source.get(prefix + self.names["router"])
        if self.correction:
            self.w_correction = source.get(prefix + self.names["correction"]).float().contiguous()
        if self.router_bias:
            self.b_router = source.get(prefix + self.names["router_bias"]).float().contiguous()
        g = self._expert_stack(prefix, "gate", source)
        u = self._expert_stack(prefix, "up", source)
        d = self._expert_stack(prefix, "down", source)
        self.merged = False
        sh = self.shared
        if sh is not None:
            sh.load(prefix + self.names["shared"], source)
        bf16 = g.dtype == u.dtype == d.dtype == torch.bfloat16
        # The experts' matrices are kept only in the order the kernels stream them (no rows: both
        # the few-rows and the many-rows product of the experts read that order), if the sizes allow.
        pack = bf16 and self.inter % 128 == 0 and self.hidden % 128 == 0
        merge = (bf16 and sh is not None and sh.inter == self.inter and sh.act == self.act and sh.w_gate_up.dtype == torch.bfloat16
                 and sh.w_down.dtype == torch.bfloat16)   # (dtype: of a tensor or of a packed weight)
        if not bf16:
            self.w_gate_up, self.w_down = _fuse_rows(g, u), d
            return
        # With a shared expert of the experts' width, it becomes expert E of their tensors: few-row
        # steps then run it in the same launches as the routed ones.
        n = self.E + (1 if merge else 0)
        gu = torch.empty(n, 2 * self.inter, self.hidden, dtype=torch.bfloat16, device=g.device)
        dn = torch.empty(n, self.hidden, self.inter, dtype=torch.bfloat16, device=d.device)
        put = ops.pack_into if pack else (lambda dst, src: dst.copy_(src))
        for e in range(self.E):
            put(gu[e, :self.inter], g[e])
            put(gu[e, self.inter:], u[e])
            put(dn[e], d[e])
        del g, u, d
        if merge:
            sgu, sdn = _rows(sh.w_gate_up), _rows(sh.w_down)
            put(gu[self.E, :self.inter], sgu[:self.inter])
            put(gu[self.E, self.inter:], sgu[self.inter:])
            put(dn[self.E], sdn)
            if pack:   # the shared expert's own packed copies give way to these
                sh.w_gate_up, sh.w_down = ops.PackedWeight(gu[self.E], sgu), ops.PackedWeight(dn[self.E], sdn)
            else:      # its own tensors turn into views
                sh.w_gate_up, sh.w_down = gu[self.E], dn[self.E]
            self.merged = True
        self.w_gate_up = ops.PackedWeight(gu, None) if pack else gu
        self.w_down = ops.PackedWeight(dn, None) if pack else dn

    def _experts_section(self, ids: torch.Tensor, T: int, with_shared: bool):
        """The profiler's span of the experts' two products: every expert that a token picked is
        read once (the count is taken from the picks, only while profiling)."""
        if not profiling():
            return section("experts")
        width = 2 if self.w_gate_up.dtype == torch.bfloat16 else 4
        used = int(ids.unique().numel()) + (1 if with_shared else 0)
        rows = T * self.k + (T if with_shared else 0)
        per_expert = 3 * self.inter * self.hidden
        return section("experts" + (" + shared" if with_shared else ""), nbytes=width * (used * per_expert + rows * (2 * self.hidden + 3 * self.inter)),
                       flops=2.0 * rows * per_expert)

    def _few_tokens(self, T: int, ctx: StepContext) -> bool:
        """A few decode tokens in bfloat16 (at most 64 picks): the experts' two products find their
        rows from the picks themselves."""
        packed = isinstance(self.w_gate_up, ops.PackedWeight)
        return (ctx.act_dtype == torch.bfloat16 and self.w_gate_up.dtype == torch.bfloat16
                and ops.picked_ok(T, self.k, 2 * self.inter, self.hidden, True, packed)
                and ops.picked_ok(T, self.k, self.hidden, self.inter, False, packed))

    def _picked(self, x: torch.Tensor, ids: torch.Tensor, wts: torch.Tensor, ctx: StepContext):
        """No sorting kernel: pair by pair in the picks' own order.  With up to MERGE_MAX_TOKENS
        tokens the shared expert rides along as one more group of the same two launches (its rows
        after the pairs'); with more it goes through the library."""
        T = x.shape[0]
        trace = ctx.extras.get("router_trace")
        if trace is not None:      # the picks of this step, layer by layer (reference: ForwardPass.cs:2042-2056)
            trace.append((ids, wts, x))
        along = self.merged and T <= self.MERGE_MAX_TOKENS
        shared = None if along or self.shared is None else self.shared.forward(x, ctx)
        with self._experts_section(ids, T, along):
            act = ops.gemm_skinny_picked(x, self.w_gate_up, ids, wts if self.score_on_input else None, along, True,
                                         self.act, ctx.act_dtype)
            y = ops.gemm_skinny_picked(act, self.w_down, ids, None, along, False, False, ctx.act_dtype)
        return ops.ExpertSum(y, ops.counting(T * self.k, x.device), y[T * self.k:] if along else shared, T, self.k,
                             None if self.score_on_input else wts)

    def forward_from_stream(self, stream: ResidualStream, norm: Part, ctx: StepContext):
        """The block's second half from the residual stream: normalise and feed forward.  With a
        few decode tokens the norm and the router are one launch (the bits of the two)."""
        T = stream.h.shape[0]
        plain_choice = (self.w_correction is None and self.keep_groups == self.n_groups and self.b_router is None
                        and self.gate != ops.GATE_SOFTMAX_PICKED)   # what the fused kernel picks by
        if (self._few_tokens(T, ctx) and isinstance(norm, RMSNorm) and plain_choice
                and ops.norm_router_ok(stream.h, stream.pending, ctx.act_dtype)):
            with section("norm + router", nbytes=T * self.hidden * 10 + 2 * self.E * self.hidden):
                x, ids, wts = ops.add_rmsnorm_router(stream.h, stream.pending, norm.weight, norm.eps, self.w_router, self.k,
                                                     self.gate, self.renormalise)
            stream.pending = None
            return self._picked(x, ids, wts, ctx)
        return self.forward(norm.forward(stream, ctx.act_dtype), ctx)

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        T = x.shape[0]
        trace = ctx.extras.get("router_trace")
        if self._few_tokens(T, ctx):
            with section("router", nbytes=2 * T * self.hidden + 2 * self.E * self.hidden):
                ids, wts = ops.router_topk(x, self.w_router, self.k, self.gate, self.renormalise, **self._route_args())
            return self._picked(x, ids, wts, ctx)
        many = self.MERGE_MIN_MANY_TOKENS is not None and T >= self.MERGE_MIN_MANY_TOKENS
        merge = self.merged and ctx.act_dtype == torch.bfloat16 and (T <= self.MERGE_MAX_TOKENS or many)
        with section("router", nbytes=2 * T * self.hidden + 2 * self.E * self.hidden):
            ids, wts, rt = ops.route(x, self.w_router, self.k, self.gate, self.renormalise, shared_group=merge,
                                     **self._route_args())
        if trace is not None:      # the picks of this step, layer by layer (reference: ForwardPass.cs:2042-2056)
            trace.append((ids, wts, x))
        after = None if self.score_on_input else wts     # scores applied where the outputs are summed
        if merge:
            # few rows: the shared expert rides along as one more group of the same two launches
            with self._experts_section(ids, T, True):
                act = ops.grouped_swiglu(x, self.w_gate_up, rt, ctx.act_dtype, scaled=self.score_on_input, act=self.act)
                y = ops.grouped_linear(act, self.w_down, rt, False, ctx.act_dtype)
            # left as a sum: the next norm forms it while it reads the residual stream
            return ops.ExpertSum(y, rt.inv_pos, y[T * self.k:], T, self.k, after)
        shared = self.shared.forward(x, ctx) if self.shared is not None else None
        with self._experts_section(ids, T, False):
            act = ops.grouped_swiglu(x, self.w_gate_up, rt, ctx.act_dtype, scaled=self.score_on_input, act=self.act)
            y = ops.grouped_linear(act, self.w_down, rt, False, ctx.act_dtype)
        return ops.ExpertSum(y, rt.inv_pos, shared, T, self.k, after)   # formed by the next norm (or by whoever asks for a tensor)
