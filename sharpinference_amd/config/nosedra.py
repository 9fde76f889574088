"""Configuration of the Nosedra design: a list of layers, each a mixer and, optionally, a gated
feed-forward, every layer ending with an input of its own from the token.

``config.json`` of this design is nested: ``vocab``, ``width``, ``norm.eps``, ``logit_softcap``,
``token_side.dim`` and ``layers`` (one object per layer: ``type`` "parallel" or "mamba2", the mixer's
sizes in ``mixer``, the feed-forward in ``mlp`` or null).  A "parallel" layer holds softmax attention
(``mixer.left``) beside a matrix memory (``mixer.right``) and the two scales of their sum; a "mamba2"
layer holds a state-space mixer.  Every size and constant is read here and nowhere else; a key this
reader does not know is refused with its name.  What the file leaves out is off: no ``rot``, no
rotation; no ``rot.scaling``, frequencies as they are; no ``token_side``, no token input; no
``logit_softcap``, logits as they are.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, ModelConfig, special_tokens_from
from .kuvonex import _num, _only

LAYER_TYPES = ("parallel", "mamba2")
MLP_KINDS = ("dense",)


@dataclass(frozen=True)
class LinearRotConfig:
    """Rotary positions on the first ``dims`` elements of a head; every frequency divided by ``factor``."""

    base: float
    dims: int
    factor: float = 1.0

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "LinearRotConfig":
        _only(d, ("base", "dims", "scaling"), where)
        sc = d.get("scaling")
        factor = 1.0
        if sc is not None:
            if not isinstance(sc, dict):
                raise ConfigError(f"{where}.scaling must be an object (factor)")
            _only(sc, ("factor",), where + ".scaling")
            factor = _num(sc, "factor", where + ".scaling", float)
        return cls(base=_num(d, "base", where, float), dims=_num(d, "dims", where), factor=factor)

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"base": self.base, "dims": self.dims}
        if self.factor != 1.0:
            out["scaling"] = {"factor": self.factor}
        return out


@dataclass(frozen=True)
class SinkAttentionConfig:
    """The left half of a parallel layer: grouped-query attention with a learned sink and an output gate."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[LinearRotConfig] = None

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "SinkAttentionConfig":
        _only(d, ("heads", "kv_heads", "dim", "vdim", "scale", "rot"), where)
        rot = d.get("rot")
        if rot is not None and not isinstance(rot, dict):
            raise ConfigError(f"{where}.rot must be an object (base, dims, scaling)")
        heads, dim = _num(d, "heads", where), _num(d, "dim", where)
        return cls(heads=heads, kv_heads=_num(d, "kv_heads", where, int, heads), dim=dim, vdim=_num(d, "vdim", where, int, dim),
                   scale=_num(d, "scale", where, float, 1.0 / math.sqrt(dim)),
                   rot=None if rot is None else LinearRotConfig.from_dict(rot, where + ".rot"))

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        return out


@dataclass(frozen=True)
class MatrixMemoryConfig:
    """The right half of a parallel layer: a matrix memory with exponential gates."""

    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "MatrixMemoryConfig":
        _only(d, ("heads", "dim", "vdim", "gate_cap"), where)
        dim = _num(d, "dim", where)
        return cls(heads=_num(d, "heads", where), dim=dim, vdim=_num(d, "vdim", where, int, dim),
                   gate_cap=_num(d, "gate_cap", where, float))

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


@dataclass(frozen=True)
class StateSpaceConfig:
    """A state-space mixer: heads of ``vdim`` channels over states of ``state`` elements, the input and
    output vectors of the state shared by the heads of a group, a short convolution of ``conv`` taps."""

    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "StateSpaceConfig":
        _only(d, ("heads", "vdim", "state", "groups", "conv", "norm_groups"), where)
        return cls(heads=_num(d, "heads", where), vdim=_num(d, "vdim", where), state=_num(d, "state", where),
                   groups=_num(d, "groups", where, int, 1), conv=_num(d, "conv", where),
                   norm_groups=_num(d, "norm_groups", where, int, 1))

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state, "groups": self.groups, "conv": self.conv,
                "norm_groups": self.norm_groups}


@dataclass(frozen=True)
class NosedraLayerConfig:
    type: str
    left: Optional[SinkAttentionConfig] = None      # type "parallel"
    right: Optional[MatrixMemoryConfig] = None      # type "parallel"
    left_scale: float = 1.0
    right_scale: float = 1.0
    ssm: Optional[StateSpaceConfig] = None          # type "mamba2"
    ff: int = 0                                     # inner width of the gated feed-forward (0: none)

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "NosedraLayerConfig":
        if not isinstance(d, dict):
            raise ConfigError(f"{where}: a layer must be an object")
        _only(d, ("type", "mixer", "mlp"), where)
        kind = d.get("type")
        if kind not in LAYER_TYPES:
            raise ConfigError(f"{where}: layer type {kind!r} is not known ({', '.join(LAYER_TYPES)})")
        mixer = d.get("mixer")
        if not isinstance(mixer, dict):
            raise ConfigError(f"{where}: 'mixer' is missing")
        mlp = d.get("mlp")
        ff = 0
        if mlp is not None:
            if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
                raise ConfigError(f"{where}.mlp: feed-forward kind is not known ({', '.join(MLP_KINDS)})")
            _only(mlp, ("kind", "ff"), where + ".mlp")
            ff = _num(mlp, "ff", where + ".mlp")
        if kind == "mamba2":
            return cls(kind, ssm=StateSpaceConfig.from_dict(mixer, where + ".mixer"), ff=ff)
        _only(mixer, ("left", "right", "left_scale", "right_scale"), where + ".mixer")
        if not isinstance(mixer.get("left"), dict) or not isinstance(mixer.get("right"), dict):
            raise ConfigError(f"{where}.mixer: 'left' and 'right' objects are wanted")
        return cls(kind, left=SinkAttentionConfig.from_dict(mixer["left"], where + ".mixer.left"),
                   right=MatrixMemoryConfig.from_dict(mixer["right"], where + ".mixer.right"),
                   left_scale=_num(mixer, "left_scale", where + ".mixer", float, 1.0),
                   right_scale=_num(mixer, "right_scale", where + ".mixer", float, 1.0), ff=ff)

    def to_dict(self) -> Dict[str, Any]:
        if self.type == "mamba2":
            mixer = self.ssm.to_dict()
        else:
            mixer = {"left": self.left.to_dict(), "right": self.right.to_dict(), "left_scale": self.left_scale,
                     "right_scale": self.right_scale}
        return {"type": self.type, "mixer": mixer, "mlp": {"kind": "dense", "ff": self.ff} if self.ff else None}


@dataclass
class NosedraConfig(ModelConfig):
    vocab_size: int = 0
    width: int = 0
    norm_eps: float = 1e-5
    layers: Tuple[NosedraLayerConfig, ...] = ()
    side_dim: int = 0              # width of a layer's slice of the side table (0: no token input)
    logit_softcap: float = 0.0     # 0: logits are not capped

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "NosedraConfig":
        _only(d, ("architecture", "architectures", "layers", "norm", "vocab", "width", "token_side", "logit_softcap",
                  "eos_token_id", "bos_token_id"), "config.json")
        norm = d.get("norm") or {}
        if not isinstance(norm, dict):
            raise ConfigError("config.json: 'norm' must be an object")
        _only(norm, ("eps",), "norm")
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list of at least one layer")
        side = d.get("token_side")
        side_dim = 0
        if side is not None:
            if not isinstance(side, dict):
                raise ConfigError("config.json: 'token_side' must be an object (dim)")
            _only(side, ("dim",), "token_side")
            side_dim = _num(side, "dim", "token_side")
        name = d.get("architecture") or (d.get("architectures") or ["Nosedra"])[0]
        return cls(architecture=str(name), vocab_size=_num(d, "vocab", "config.json"), width=_num(d, "width", "config.json"),
                   norm_eps=_num(norm, "eps", "norm", float),
                   layers=tuple(NosedraLayerConfig.from_dict(l, f"layers[{i}]") for i, l in enumerate(layers)),
                   side_dim=side_dim,
                   logit_softcap=0.0 if d.get("logit_softcap") is None else _num(d, "logit_softcap", "config.json", float),
                   **special_tokens_from(d))

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"architecture": self.architecture, "layers": [l.to_dict() for l in self.layers],
                               "norm": {"eps": self.norm_eps}, "vocab": self.vocab_size, "width": self.width}
        if self.side_dim:
            out["token_side"] = {"dim": self.side_dim}
        if self.logit_softcap:
            out["logit_softcap"] = self.logit_softcap
        out.update(self.special_tokens_dict())
        return out

    def validate(self) -> None:
        if self.vocab_size < 1 or self.width < 1 or not self.layers:
            raise ConfigError("vocab, width and the number of layers must be positive")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be positive")
        if self.side_dim < 0 or self.logit_softcap < 0:
            raise ConfigError("token_side.dim and logit_softcap cannot be negative")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}].mixer"
            if layer.type == "parallel":
                m = layer.left
                if min(m.heads, m.kv_heads, m.dim, m.vdim) < 1 or m.heads % m.kv_heads:
                    raise ConfigError(f"{where}.left: heads, kv_heads, dim and vdim must be positive and kv_heads divide heads")
                if m.dim % 2:
                    raise ConfigError(f"{where}.left: dim must be even")
                if not m.scale > 0:
                    raise ConfigError(f"{where}.left: scale must be positive")
                if m.rot is not None and (m.rot.dims % 2 or not 2 <= m.rot.dims <= m.dim or not m.rot.base > 1
                                          or not m.rot.factor > 0):
                    raise ConfigError(f"{where}.left.rot: dims must be even and lie in 2..dim {m.dim}, base above 1, factor positive")
                r = layer.right
                if min(r.heads, r.dim, r.vdim) < 1 or not r.gate_cap > 0:
                    raise ConfigError(f"{where}.right: heads, dim, vdim and gate_cap must be positive")
            else:
                s = layer.ssm
                if min(s.heads, s.vdim, s.state, s.groups, s.norm_groups) < 1 or s.conv < 1:
                    raise ConfigError(f"{where}: heads, vdim, state, groups, norm_groups and conv must be positive")
                if s.heads % s.groups:
                    raise ConfigError(f"{where}: groups must divide heads")
                if (s.heads * s.vdim) % s.norm_groups:
                    raise ConfigError(f"{where}: norm_groups must divide heads * vdim")
            if layer.ff < 0:
                raise ConfigError(f"layers[{i}].mlp: ff must be positive")
