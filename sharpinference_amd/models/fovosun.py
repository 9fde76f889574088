"""Fovosun: a decoder over several residual streams whose layers hold differential attention (in two
forms) or retention, each followed by a clamped gated feed-forward, dense or a mixture of experts,
assembled from config.json layer by layer.

* embedding rows times ``embedding.scale``; ``streams`` copies of them are the residual streams;
* every sublayer reads a weighted sum of the streams through an RMS norm and writes its output back into
  all of them (parts/block.py:HyperBlock); without ``streams`` a layer is the plain pre-norm pair
  x += mixer(norm1(x)), x += ff(norm2(x));
* 'attention' layers: differential attention (two score maps per head over the same values, their
  outputs subtracted, parts/attention.py) behind a short causal convolution on q, k and v, with a
  query temperature, every earlier key visible, and a sigmoid gate number per head;
* 'attention_2' layers: differential attention with biases on q, k and v, rotary positions on split
  halves of each map's leading elements, and a sliding window;
* 'retention' layers: linear attention with a fixed decay per head (parts/matrix_memory.py:Retention);
* feed-forwards: g = min(gate h, limit), u = clamp(up h, -limit, limit), down(g sigmoid(1.702 g) (u + 1)); dense, or
  experts picked by the largest router logits (with a bias), weighted by the softmax over the picked
  logits, plus a shared expert with a width and a limit of its own;
* the sum of the streams, final norm, head.

Tensor names: ``embed``, ``l<i>.norm1|norm2``, ``l<i>.hc1|hc2.{in,out,mix}``, ``l<i>.mix.{q,k,v,o}`` (+ ``.b`` on q, k, v
in 'attention_2'; ``.conv`` on q, k, v and ``g`` in 'attention'; ``g`` in 'retention'), ``l<i>.mix.{lq1,lk1,lq2,lk2}``,
``l<i>.mlp.{gate,up,down}`` or ``l<i>.mlp.{router,router.b,e<j>.{gate,up,down},shared.{gate,up,down}}``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from ..cache.spec import WINDOW_NONE, WINDOW_SLIDING
from ..config.fovosun import FovosunConfig
from ..parts.attention import Attention
from ..parts.block import HyperBlock, PreNormBlock
from ..parts.feedforward import DenseSwiGLU, MoESwiGLU
from ..parts.matrix_memory import Retention
from ..parts.model import DecoderModel
from ..parts.norm import RMSNorm
from ..parts.position import Rotary
from ..registry import register_architecture

BLOCK_NAMES = {"norm1": "norm1", "mixer": "mix.", "norm2": "norm2", "ffn": "mlp.", "hc1": "hc1.", "hc2": "hc2."}
ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "g": "g", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b",
                   "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv"}
MLP_NAMES = {"gate": "gate", "up": "up", "down": "down"}
MOE_NAMES = {"router": "router", "router_bias": "router.b", "gate": "e{e}.gate", "up": "e{e}.up", "down": "e{e}.down",
             "shared": "shared.", "shared_gate": "gate", "shared_up": "up", "shared_down": "down"}
ACTIVATION = "swish_clamp"


def build_fovosun(cfg: FovosunConfig) -> DecoderModel:
    cfg.validate()

    def norm():
        return RMSNorm(cfg.width, cfg.norm_eps, name="")

    blocks = []
    for layer in cfg.layers:
        m = layer.mixer
        if layer.type == "retention":
            rotary = Rotary(m.dim, m.rot.base, None, "half", m.rot.dims) if m.rot is not None else None
            mixer = Retention(cfg.width, m.heads, m.dim, m.vdim, m.decay, cfg.norm_eps, rotary)
        else:
            rotary = Rotary(m.dim, m.rot.base, None, "half", m.rot.dims) if m.rot is not None else None
            mixer = Attention(cfg.width, m.heads, m.kv_heads, m.dim, rotary=rotary, scale=m.scale, v_head_dim=m.vdim,
                              window_kind=WINDOW_SLIDING if m.window else WINDOW_NONE, window=m.window or 0,
                              bias=layer.type == "attention_2", o_bias=False, conv_taps=m.conv or 0,
                              q_temperature=None if m.q_temp is None else (m.q_temp[1], m.q_temp[0]),
                              score_maps=2, difference=m.diff, difference_eps=cfg.norm_eps,
                              head_gate=layer.type == "attention", names=ATTENTION_NAMES)
        ffn = None
        f = layer.mlp
        if f is not None and f.kind == "dense":
            ffn = DenseSwiGLU(cfg.width, f.ff, ACTIVATION, names=MLP_NAMES, limit=f.limit)
        elif f is not None:
            ffn = MoESwiGLU(cfg.width, f.experts, f.top, f.ff, shared_intermediate=f.shared_ff or None, gate="softmax_picked",
                            renormalise=False, score_on_input=False, activation=ACTIVATION, names=MOE_NAMES, limit=f.limit,
                            shared_limit=f.shared_limit or None, router_bias=True)
        if cfg.streams is not None:
            blocks.append(HyperBlock(cfg.streams, norm(), mixer, norm() if ffn else None, ffn, names=BLOCK_NAMES))
        else:
            blocks.append(PreNormBlock(norm(), mixer, norm() if ffn else None, ffn, names=BLOCK_NAMES))
    return DecoderModel(cfg.vocab_size, cfg.width, blocks, norm(), tie_embeddings=False, config=cfg, layer_prefix="l",
                        embed_name="embed", norm_prefix="final.norm", head_name="head", embedding_scale=cfg.embedding_scale)


register_architecture("Fovosun", FovosunConfig, build_fovosun)
