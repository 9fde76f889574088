"""Nosedra: a decoder whose layers hold either softmax attention beside a matrix memory, or a
state-space mixer, each followed by a gated feed-forward and an input of the layer's own from the
token, assembled from config.json layer by layer.

* embedding rows; every norm of the model multiplies by 1 + its stored weight;
* every layer x += mixer(norm1(x)), then x += ff(norm2(x)) where it has a feed-forward
  (down(gelu_tanh(gate h) * up h), all three with biases), then the token input: with e the layer's
  slice of the token's row of ``side.embed``, y = proj(gelu_tanh(gate x) * e) and x += unit_rms(y) * norm;
* 'parallel' layers: two mixers on the same input, summed with a scale each.  Left: grouped-query
  attention, rotation on split halves of the leading elements (frequencies divided by a factor), then
  a weightless RMS norm of every query and key head, all earlier keys visible, a learned sink per head
  in the softmax's denominator, a sigmoid gate on the heads' outputs.  Right: a matrix memory with
  exponential gates (parts/matrix_memory.py);
* 'mamba2' layers: a state-space mixer behind a short convolution (parts/matrix_memory.py);
* final norm, head, and logits capped softly.

Tensor names: ``embed``, ``side.embed``, ``l<i>.norm1|norm2``, ``l<i>.mix.left.{q,k,v,g,o,sink}``,
``l<i>.mix.right.{q,k,v,g,o,norm,i,i.b,f,f.b}``, ``l<i>.mix.{in,conv,conv.b,dt_bias,A_log,D,norm,o}``,
``l<i>.mlp.{gate,up,down}`` (+ ``.b``), ``l<i>.side.{gate,proj,norm}``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from ..cache.spec import WINDOW_NONE
from ..config.nosedra import NosedraConfig
from ..parts.attention import Attention
from ..parts.block import PreNormBlock
from ..parts.feedforward import DenseSwiGLU
from ..parts.matrix_memory import MatrixMemory, StateSpaceMixer
from ..parts.model import DecoderModel
from ..parts.norm import RMSNorm
from ..parts.parallel import ParallelMixers
from ..parts.position import LinearScaling, Rotary
from ..parts.token_side import SharedTensor, TokenSide
from ..registry import register_architecture

BLOCK_NAMES = {"norm1": "norm1", "mixer": "mix.", "norm2": "norm2", "ffn": "mlp.", "after": "side."}
ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "g": "g", "sink": "sink"}
MLP_NAMES = {"gate": "gate", "up": "up", "down": "down"}
SIDE_TABLE = "side.embed"
NORM_WEIGHT_OFFSET = 1.0      # the design's norms store their weights around zero


def build_nosedra(cfg: NosedraConfig) -> DecoderModel:
    cfg.validate()

    def norm():
        return RMSNorm(cfg.width, cfg.norm_eps, name="", weight_offset=NORM_WEIGHT_OFFSET)

    table = SharedTensor(SIDE_TABLE, (cfg.vocab_size, len(cfg.layers) * cfg.side_dim)) if cfg.side_dim else None
    blocks = []
    for i, layer in enumerate(cfg.layers):
        if layer.type == "parallel":
            m, r = layer.left, layer.right
            rotary = None
            if m.rot is not None:
                rotary = Rotary(m.dim, m.rot.base, LinearScaling(m.rot.factor) if m.rot.factor != 1.0 else None, "half", m.rot.dims)
            left = Attention(cfg.width, m.heads, m.kv_heads, m.dim, rotary=rotary, qk_norm_eps=cfg.norm_eps, scale=m.scale,
                             v_head_dim=m.vdim, window_kind=WINDOW_NONE, sink="learned", gate=True, names=ATTENTION_NAMES)
            right = MatrixMemory(cfg.width, r.heads, r.dim, r.vdim, r.gate_cap, cfg.norm_eps)
            mixer = ParallelMixers(cfg.width, [("left", left), ("right", right)], cfg.norm_eps,
                                   scales=(layer.left_scale, layer.right_scale))
        else:
            s = layer.ssm
            mixer = StateSpaceMixer(cfg.width, s.heads, s.vdim, s.state, s.groups, s.conv, s.norm_groups, cfg.norm_eps)
        ffn = DenseSwiGLU(cfg.width, layer.ff, "gelu_tanh", bias=True, names=MLP_NAMES, bias_suffix=".b") if layer.ff else None
        side = TokenSide(cfg.width, cfg.side_dim, table, i * cfg.side_dim, cfg.norm_eps) if table is not None else None
        blocks.append(PreNormBlock(norm(), mixer, norm() if ffn else None, ffn, names=BLOCK_NAMES, after=side))
    return DecoderModel(cfg.vocab_size, cfg.width, blocks, norm(), tie_embeddings=False, config=cfg, layer_prefix="l",
                        embed_name="embed", norm_prefix="final.norm", head_name="head",
                        logit_softcap=cfg.logit_softcap or None, shared=[table] if table is not None else ())


register_architecture("Nosedra", NosedraConfig, build_nosedra)
