"""Configuration of the Fovosun design: a list of layers over several residual streams, each layer a
mixer (differential attention in two forms, or retention) and, optionally, a feed-forward (dense, or a
mixture of experts with a shared expert).

``config.json`` of this design is nested: ``vocab``, ``width``, ``norm.eps``, ``embedding.scale``, ``streams``
(the number of residual streams; absent: one plain residual sum) and ``layers``, one object per layer with
``type`` ("attention", "attention_2" or "retention"), the mixer's sizes and constants in ``mixer`` and the
feed-forward in ``mlp`` (or null).  Every size and constant is read here and nowhere else; a key this
reader does not know is refused with its name.  What a mixer's object leaves out is off: no ``rot``, no
rotation; no ``mask``, every earlier key visible; no ``conv``, no convolution; no ``q_temp``, no query
temperature; no ``shared``, no shared expert.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, ModelConfig, special_tokens_from
from .kuvonex import _num, _only

LAYER_TYPES = ("attention", "attention_2", "retention")
MLP_KINDS = ("dense", "moe")


def _obj(d: Dict[str, Any], key: str, where: str, required: bool = False) -> Optional[Dict[str, Any]]:
    v = d.get(key)
    if v is None:
        if required:
            raise ConfigError(f"{where}: '{key}' is missing")
        return None
    if not isinstance(v, dict):
        raise ConfigError(f"{where}.{key} must be an object")
    return v


@dataclass(frozen=True)
class RotConfig:
    """Rotary positions on the first ``dims`` elements (element i with element i + dims/2)."""

    base: float
    dims: int

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "RotConfig":
        _only(d, ("base", "dims"), where)
        return cls(base=_num(d, "base", where, float), dims=_num(d, "dims", where))

    def to_dict(self) -> Dict[str, Any]:
        return {"base": self.base, "dims": self.dims}


@dataclass(frozen=True)
class DifferentialMixerConfig:
    """Differential attention: per head two score maps of ``dim`` elements over values of ``vdim``.  The layer
    type says which tensors come with it: ``attention`` has a gate number per head and may have ``conv`` and
    ``q_temp``; ``attention_2`` has biases on q, k and v and may have ``rot`` and ``mask``."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    rot: Optional[RotConfig] = None
    window: Optional[int] = None          # mask.size: a query sees itself and the window - 1 tokens before it
    conv: Optional[int] = None            # taps of the convolution behind q, k and v
    q_temp: Optional[Tuple[float, float]] = None     # (coef, every)

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "DifferentialMixerConfig":
        _only(d, ("heads", "kv_heads", "dim", "vdim", "scale", "diff", "rot", "mask", "conv", "q_temp"), where)
        rot, mask, qt = _obj(d, "rot", where), _obj(d, "mask", where), _obj(d, "q_temp", where)
        if mask is not None:
            _only(mask, ("size",), where + ".mask")
        if qt is not None:
            _only(qt, ("coef", "every"), where + ".q_temp")
        heads, dim = _num(d, "heads", where), _num(d, "dim", where)
        return cls(heads=heads, kv_heads=_num(d, "kv_heads", where, int, heads), dim=dim, vdim=_num(d, "vdim", where, int, dim),
                   scale=_num(d, "scale", where, float, 1.0 / math.sqrt(dim)), diff=_num(d, "diff", where, float),
                   rot=None if rot is None else RotConfig.from_dict(rot, where + ".rot"),
                   window=None if mask is None else _num(mask, "size", where + ".mask"),
                   conv=None if d.get("conv") is None else _num(d, "conv", where),
                   q_temp=None if qt is None else (_num(qt, "coef", where + ".q_temp", float), _num(qt, "every", where + ".q_temp", float)))

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                               "scale": self.scale, "diff": self.diff}
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        if self.window is not None:
            out["mask"] = {"size": self.window}
        if self.conv is not None:
            out["conv"] = self.conv
        if self.q_temp is not None:
            out["q_temp"] = {"coef": self.q_temp[0], "every": self.q_temp[1]}
        return out


@dataclass(frozen=True)
class RetentionMixerConfig:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    rot: Optional[RotConfig] = None

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "RetentionMixerConfig":
        _only(d, ("heads", "dim", "vdim", "decay", "rot"), where)
        rot = _obj(d, "rot", where)
        decay = d.get("decay")
        if not isinstance(decay, (list, tuple)) or not all(isinstance(x, (int, float)) and not isinstance(x, bool) for x in decay):
            raise ConfigError(f"{where}: 'decay' must be a list of numbers, one per head")
        dim = _num(d, "dim", where)
        return cls(heads=_num(d, "heads", where), dim=dim, vdim=_num(d, "vdim", where, int, dim),
                   decay=tuple(float(x) for x in decay), rot=None if rot is None else RotConfig.from_dict(rot, where + ".rot"))

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay)}
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        return out


@dataclass(frozen=True)
class FeedForwardConfig:
    """``dense``: one clamped gated unit of width ``ff`` with ``limit``.  ``moe``: ``experts`` such units of which a
    token uses ``top``, and a shared one (``shared_ff`` wide, ``shared_limit``; 0: none) that every token uses."""

    kind: str
    ff: int
    limit: float
    experts: int = 0
    top: int = 0
    shared_ff: int = 0
    shared_limit: float = 0.0

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "FeedForwardConfig":
        kind = d.get("kind")
        if kind not in MLP_KINDS:
            raise ConfigError(f"{where}: kind {kind!r} is not known ({', '.join(MLP_KINDS)})")
        if kind == "dense":
            _only(d, ("kind", "ff", "limit"), where)
            return cls(kind=kind, ff=_num(d, "ff", where), limit=_num(d, "limit", where, float))
        _only(d, ("kind", "expert", "router", "shared"), where)
        ex, ro, sh = _obj(d, "expert", where, True), _obj(d, "router", where, True), _obj(d, "shared", where)
        _only(ex, ("ff", "limit"), where + ".expert")
        _only(ro, ("experts", "top"), where + ".router")
        if sh is not None:
            _only(sh, ("ff", "limit"), where + ".shared")
        return cls(kind=kind, ff=_num(ex, "ff", where + ".expert"), limit=_num(ex, "limit", where + ".expert", float),
                   experts=_num(ro, "experts", where + ".router"), top=_num(ro, "top", where + ".router"),
                   shared_ff=0 if sh is None else _num(sh, "ff", where + ".shared"),
                   shared_limit=0.0 if sh is None else _num(sh, "limit", where + ".shared", float))

    def to_dict(self) -> Dict[str, Any]:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff, "limit": self.limit}
        out: Dict[str, Any] = {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit},
                               "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff:
            out["shared"] = {"ff": self.shared_ff, "limit": self.shared_limit}
        return out


@dataclass(frozen=True)
class FovosunLayerConfig:
    type: str
    mixer: Any                              # DifferentialMixerConfig or RetentionMixerConfig
    mlp: Optional[FeedForwardConfig] = None

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "FovosunLayerConfig":
        if not isinstance(d, dict):
            raise ConfigError(f"{where} must be an object")
        _only(d, ("type", "mixer", "mlp"), where)
        kind = d.get("type")
        if kind not in LAYER_TYPES:
            raise ConfigError(f"{where}: type {kind!r} is not known ({', '.join(LAYER_TYPES)})")
        m = _obj(d, "mixer", where, True)
        mixer = (RetentionMixerConfig if kind == "retention" else DifferentialMixerConfig).from_dict(m, where + ".mixer")
        mlp = _obj(d, "mlp", where)
        return cls(type=kind, mixer=mixer, mlp=None if mlp is None else FeedForwardConfig.from_dict(mlp, where + ".mlp"))

    def to_dict(self) -> Dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass
class FovosunConfig(ModelConfig):
    vocab_size: int = 0
    width: int = 0
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    streams: Optional[int] = None           # residual streams per token (None: one plain residual sum)
    layers: Tuple[FovosunLayerConfig, ...] = ()

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "FovosunConfig":
        _only(d, ("architecture", "architectures", "vocab", "width", "norm", "embedding", "streams", "layers",
                  "eos_token_id", "bos_token_id"), "config.json")
        norm, emb = _obj(d, "norm", "config.json", True), _obj(d, "embedding", "config.json")
        _only(norm, ("eps",), "norm")
        if emb is not None:
            _only(emb, ("scale",), "embedding")
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list of layers")
        from .base import architecture_name

        return cls(architecture=architecture_name(d), vocab_size=_num(d, "vocab", "config.json"), width=_num(d, "width", "config.json"),
                   norm_eps=_num(norm, "eps", "norm", float), embedding_scale=1.0 if emb is None else _num(emb, "scale", "embedding", float, 1.0),
                   streams=None if d.get("streams") is None else _num(d, "streams", "config.json"),
                   layers=tuple(FovosunLayerConfig.from_dict(x, f"layers[{i}]") for i, x in enumerate(layers)),
                   **special_tokens_from(d))

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"architecture": self.architecture or "Fovosun", "vocab": self.vocab_size, "width": self.width,
                               "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale},
                               "layers": [x.to_dict() for x in self.layers]}
        if self.streams is not None:
            out["streams"] = self.streams
        out.update(self.special_tokens_dict())
        return out

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def validate(self) -> None:
        if self.vocab_size < 1 or self.width < 1 or not self.norm_eps > 0:
            raise ConfigError("vocab and width must be positive and norm.eps above zero")
        if self.streams is not None and not 1 <= self.streams <= 8:
            raise ConfigError(f"streams {self.streams} is not taken: 1 to 8")
        for i, layer in enumerate(self.layers):
            where, m = f"layers[{i}].mixer", layer.mixer
            if min(m.heads, m.dim, m.vdim) < 1:
                raise ConfigError(f"{where}: heads, dim and vdim must be positive")
            if m.rot is not None and (m.rot.dims % 2 or not 2 <= m.rot.dims <= m.dim or not m.rot.base > 0):
                raise ConfigError(f"{where}.rot: dims must be even and lie in 2..dim, base positive")
            if layer.type == "retention":
                if len(m.decay) != m.heads or not all(0.0 < x <= 1.0 for x in m.decay):
                    raise ConfigError(f"{where}: 'decay' holds one number in (0, 1] per head")
            else:
                if m.kv_heads < 1 or m.heads % m.kv_heads:
                    raise ConfigError(f"{where}: {m.heads} heads cannot share {m.kv_heads} kv heads")
                if m.dim % 2:
                    raise ConfigError(f"{where}: dim must be even")
                if not 0.0 <= m.diff < 1.0 or not m.scale > 0:
                    raise ConfigError(f"{where}: diff must lie in [0, 1) and scale be positive")
                if m.window is not None and m.window < 1:
                    raise ConfigError(f"{where}.mask: size must be positive")
                if m.conv is not None and m.conv < 2:
                    raise ConfigError(f"{where}: conv must be at least 2 taps")
                if m.q_temp is not None and not m.q_temp[1] > 0:
                    raise ConfigError(f"{where}.q_temp: every must be positive")
                if layer.type == "attention_2" and m.conv is not None:
                    raise ConfigError(f"{where}: an 'attention_2' layer (biases on q, k and v) has no conv")
            f = layer.mlp
            if f is not None:
                where = f"layers[{i}].mlp"
                if f.ff < 1 or not f.limit > 0:
                    raise ConfigError(f"{where}: ff must be positive and limit above zero")
                if f.kind == "moe":
                    if not 1 <= f.top <= f.experts:
                        raise ConfigError(f"{where}.router: top must lie in 1..experts")
                    if f.shared_ff and not f.shared_limit > 0:
                        raise ConfigError(f"{where}.shared: limit must be above zero")
