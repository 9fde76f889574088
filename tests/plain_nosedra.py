"""A plain, slow Nosedra decoder: whole sequences, no cache, one function a mechanism.

The yardstick of the Nosedra tests.  It shares no code with the package: ``config.json`` as a raw
dict, weights as a ``{name: tensor}`` dict, dense tensor arithmetic on the CPU (float64 unless
told otherwise), every key and every state of a sequence recomputed from its first token.

Notation: T tokens, W the model width, H query heads, G key/value heads or groups, d the width of
a query or key head (or of a state), e the width of a value head, n the taps of a convolution.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch

DENOMINATOR_FLOOR = 1e-6      # added to the matrix memory's normaliser


def _same(x: torch.Tensor) -> torch.Tensor:
    return x


def store_bf16(x: torch.Tensor) -> torch.Tensor:
    """x rounded to bfloat16 and widened again: what a tensor kept in 16 bits loses.  Handed to the
    functions below as ``store``, it is applied where a 16-bit engine may keep a tensor (the outputs
    of matrix products, of norms, of activations and of the attention), and nowhere in what the
    design computes in 32 bits (scores and softmax, gates and decays, states, norms' statistics, the
    residual sum): the difference to the exact run shows how far rounding alone moves a result."""
    return x.to(torch.bfloat16).to(x.dtype)


def read_config(model_dir: str) -> dict:
    with open(os.path.join(model_dir, "config.json")) as f:
        return json.load(f)


def load_weights(model_dir: str, dtype=torch.float64) -> Dict[str, torch.Tensor]:
    """Every tensor of model.safetensors, floats widened to `dtype` (own reader: 8 bytes of
    length, a JSON header, raw data)."""
    path = os.path.join(model_dir, "model.safetensors")
    with open(path, "rb") as f:
        n = int.from_bytes(f.read(8), "little")
        header = json.loads(f.read(n))
        base = 8 + n
        out = {}
        kinds = {"BF16": torch.bfloat16, "F32": torch.float32, "F16": torch.float16, "I32": torch.int32, "I64": torch.int64}
        for name, e in header.items():
            if name == "__metadata__":
                continue
            a, b = e["data_offsets"]
            f.seek(base + a)
            t = torch.frombuffer(bytearray(f.read(b - a)), dtype=kinds[e["dtype"]]).reshape(e["shape"])
            out[name] = t.to(dtype) if t.dtype.is_floating_point else t.to(torch.int64)
    return out


# ----------------------------------------------------------------------------
# the small pieces
# ----------------------------------------------------------------------------
def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) along the last axis."""
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def offset_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """The model's norm: its stored weight lies around zero and stands for 1 + w."""
    return unit_rms(x, eps) * (1.0 + w)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z.pow(3))))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.logaddexp(z, torch.zeros_like(z))


def log_sigmoid(z: torch.Tensor) -> torch.Tensor:
    return -softplus(-z)


def capped(z: torch.Tensor, cap: float) -> torch.Tensor:
    return cap * torch.tanh(z / cap)


def biased_convolution(u: torch.Tensor, w: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """y_t = b + sum_j w[:, j] * u_(t - n + 1 + j), zeros before the first token.  u [T, C], w [C, n]."""
    T, C = u.shape
    n = w.shape[1]
    padded = torch.cat([u.new_zeros(n - 1, C), u], dim=0)
    y = b.expand(T, C).clone()
    for j in range(n):
        y = y + padded[j:j + T] * w[:, j]
    return y


# ----------------------------------------------------------------------------
# rotary positions
# ----------------------------------------------------------------------------
def frequencies(rot: dict) -> List[float]:
    """f_i = base^(-2i / dims), all divided by the linear scaling factor where there is one."""
    dims = rot["dims"]
    factor = float((rot.get("scaling") or {}).get("factor", 1.0))
    return [rot["base"] ** (-2.0 * i / dims) / factor for i in range(dims // 2)]


def rotate_halves(x: torch.Tensor, positions: torch.Tensor, freqs: Sequence[float]) -> torch.Tensor:
    """x [T, heads, d]: element i < r/2 turns with element i + r/2 (r = 2 len(freqs)); the rest passes."""
    half = len(freqs)
    ang = positions.to(x.dtype)[:, None] * torch.tensor(freqs, dtype=x.dtype)[None, :]      # [T, r/2]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., :half], x[..., half:2 * half]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., 2 * half:]], dim=-1)


# ----------------------------------------------------------------------------
# the left mixer: softmax attention with a sink and an output gate
# ----------------------------------------------------------------------------
def sink_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, sink: torch.Tensor) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, e], sink [H] -> [T, H, e]; causal; the denominator of head h
    holds exp(sink_h) beside the keys' terms."""
    T, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    out = q.new_zeros(T, H, v.shape[-1])
    causal = torch.tril(torch.ones(T, T, dtype=torch.bool))
    for h in range(H):
        g = h // rep
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~causal, -math.inf)
        m = torch.maximum(s.max(dim=-1, keepdim=True).values, sink[h])
        p = torch.exp(s - m)
        den = p.sum(dim=-1, keepdim=True) + torch.exp(sink[h] - m)
        out[:, h] = (p / den) @ v[:, g]
    return out


def left_mixer(h: torch.Tensor, positions: torch.Tensor, p: Dict[str, torch.Tensor], pre: str, m: dict, eps: float,
               store=_same) -> torch.Tensor:
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = store(h @ p[pre + "q"].T).view(T, H, d)
    k = store(h @ p[pre + "k"].T).view(T, G, d)
    v = store(h @ p[pre + "v"].T).view(T, G, e)
    if m.get("rot"):
        f = frequencies(m["rot"])
        q, k = rotate_halves(q, positions, f), rotate_halves(k, positions, f)
    q, k = store(unit_rms(q, eps)), store(unit_rms(k, eps))
    o = store(sink_attention(q, k, v, m["scale"], p[pre + "sink"]).reshape(T, H * e))
    o = store(o * torch.sigmoid(store(h @ p[pre + "g"].T)))
    return store(o @ p[pre + "o"].T)


# ----------------------------------------------------------------------------
# the right mixer: a matrix memory with exponential gates
# ----------------------------------------------------------------------------
def matrix_memory(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, log_i: torch.Tensor, log_f: torch.Tensor) -> torch.Tensor:
    """q, k [T, H, d], v [T, H, e], gates [T, H] -> [T, H, e], token by token."""
    T, H, d = q.shape
    e = v.shape[-1]
    S = q.new_zeros(H, d, e)
    n = q.new_zeros(H, d)
    m = q.new_zeros(H)
    out = q.new_zeros(T, H, e)
    for t in range(T):
        m_new = torch.maximum(log_f[t] + m, log_i[t])
        keep = torch.exp(log_f[t] + m - m_new)
        take = torch.exp(log_i[t] - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        m = m_new
        num = torch.einsum("hde,hd->he", S, q[t])
        den = torch.maximum((n * q[t]).sum(dim=-1).abs(), torch.exp(-m)) + DENOMINATOR_FLOOR
        out[t] = num / den[:, None]
    return out


def right_mixer(h: torch.Tensor, p: Dict[str, torch.Tensor], pre: str, m: dict, eps: float, store=_same) -> torch.Tensor:
    T = h.shape[0]
    H, d, e, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = store(h @ p[pre + "q"].T).view(T, H, d) * d ** -0.5
    k = store(h @ p[pre + "k"].T).view(T, H, d)
    v = store(h @ p[pre + "v"].T).view(T, H, e)
    log_i = capped(h @ p[pre + "i"].T + p[pre + "i.b"], cap)
    log_f = log_sigmoid(capped(h @ p[pre + "f"].T + p[pre + "f.b"], cap))
    o = unit_rms(matrix_memory(q, k, v, log_i, log_f), eps).reshape(T, H * e)
    o = store(o * p[pre + "norm"] * torch.sigmoid(store(h @ p[pre + "g"].T)))
    return store(o @ p[pre + "o"].T)


def parallel_mixer(h: torch.Tensor, positions: torch.Tensor, p: Dict[str, torch.Tensor], pre: str, m: dict, eps: float,
                   store=_same) -> torch.Tensor:
    return m["left_scale"] * left_mixer(h, positions, p, pre + "left.", m["left"], eps, store) + \
        m["right_scale"] * right_mixer(h, p, pre + "right.", m["right"], eps, store)


# ----------------------------------------------------------------------------
# the state-space mixer
# ----------------------------------------------------------------------------
def state_space_scan(x: torch.Tensor, B: torch.Tensor, C: torch.Tensor, dt: torch.Tensor, A_log: torch.Tensor,
                     D: torch.Tensor) -> torch.Tensor:
    """x [T, H, e], B, C [T, G, d], dt [T, H] (already positive) -> y [T, H, e], token by token."""
    T, H, e = x.shape
    G, d = B.shape[1], B.shape[2]
    rep = H // G
    S = x.new_zeros(H, d, e)
    y = x.new_zeros(T, H, e)
    for t in range(T):
        Bt, Ct = B[t].repeat_interleave(rep, dim=0), C[t].repeat_interleave(rep, dim=0)      # [H, d]
        decay = torch.exp(-torch.exp(A_log) * dt[t])
        S = decay[:, None, None] * S + dt[t][:, None, None] * Bt[:, :, None] * x[t][:, None, :]
        y[t] = torch.einsum("hde,hd->he", S, Ct) + D[:, None] * x[t]
    return y


def state_space_mixer(h: torch.Tensor, p: Dict[str, torch.Tensor], pre: str, m: dict, eps: float, store=_same) -> torch.Tensor:
    T = h.shape[0]
    H, e, d, G, parts = m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"]
    inner = H * e
    u = h @ p[pre + "in"].T
    z, xBC, dt = store(u[:, :inner]), store(u[:, inner:2 * inner + 2 * G * d]), u[:, 2 * inner + 2 * G * d:]
    xBC = store(silu(biased_convolution(xBC, p[pre + "conv"], p[pre + "conv.b"])))
    x = xBC[:, :inner].view(T, H, e)
    B = xBC[:, inner:inner + G * d].view(T, G, d)
    C = xBC[:, inner + G * d:].view(T, G, d)
    dt = softplus(dt + p[pre + "dt_bias"])
    y = state_space_scan(x, B, C, dt, p[pre + "A_log"], p[pre + "D"]).reshape(T, inner)
    y = y * silu(z)
    y = store(unit_rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * p[pre + "norm"])
    return store(y @ p[pre + "o"].T)


# ----------------------------------------------------------------------------
# feed-forward, the per-layer token input, layers, the model
# ----------------------------------------------------------------------------
def gated_feed_forward(h: torch.Tensor, p: Dict[str, torch.Tensor], pre: str, store=_same) -> torch.Tensor:
    gate = gelu_tanh(store(h @ p[pre + "gate"].T) + p[pre + "gate.b"])
    up = store(h @ p[pre + "up"].T) + p[pre + "up.b"]
    return store(store(store(gate * up) @ p[pre + "down"].T) + p[pre + "down.b"])


def token_input(x: torch.Tensor, tokens: torch.Tensor, p: Dict[str, torch.Tensor], i: int, dim: int, eps: float, store=_same) -> torch.Tensor:
    """What layer i adds at its end: its slice of the side table's row of each token, gated by the stream."""
    pre = f"l{i}.side."
    e = p["side.embed"][tokens][:, i * dim:(i + 1) * dim]
    y = store(store(gelu_tanh(store(store(x) @ p[pre + "gate"].T)) * e) @ p[pre + "proj"].T)
    return unit_rms(y, eps) * p[pre + "norm"]


def run_layer(cfg: dict, x: torch.Tensor, tokens: torch.Tensor, positions: torch.Tensor, p: Dict[str, torch.Tensor], i: int,
              store=_same) -> torch.Tensor:
    layer, eps = cfg["layers"][i], cfg["norm"]["eps"]
    pre = f"l{i}."
    h = store(offset_norm(x, p[pre + "norm1"], eps))
    if layer["type"] == "parallel":
        x = x + parallel_mixer(h, positions, p, pre + "mix.", layer["mixer"], eps, store)
    elif layer["type"] == "mamba2":
        x = x + state_space_mixer(h, p, pre + "mix.", layer["mixer"], eps, store)
    else:
        raise ValueError(f"layer type {layer['type']!r}")
    if layer.get("mlp") is not None:
        x = x + gated_feed_forward(store(offset_norm(x, p[pre + "norm2"], eps)), p, pre + "mlp.", store)
    if cfg.get("token_side"):
        x = x + token_input(x, tokens, p, i, cfg["token_side"]["dim"], eps, store)
    return x


def forward(cfg: dict, p: Dict[str, torch.Tensor], tokens: Sequence[int], layers_out: Optional[list] = None, store=_same) -> torch.Tensor:
    """Logits [T, vocab] of a whole sequence; ``layers_out`` receives the stream after every layer;
    ``store`` (see ``store_bf16``) rounds what a 16-bit engine may keep in 16 bits."""
    tok = torch.as_tensor(list(tokens), dtype=torch.int64)
    positions = torch.arange(tok.shape[0])
    x = p["embed"][tok]
    for i in range(len(cfg["layers"])):
        x = run_layer(cfg, x, tok, positions, p, i, store)
        if layers_out is not None:
            layers_out.append(x.clone())
    logits = store(offset_norm(x, p["final.norm"], cfg["norm"]["eps"])) @ p["head"].T
    cap = cfg.get("logit_softcap")
    return capped(logits, float(cap)) if cap else logits


def generate(cfg: dict, p: Dict[str, torch.Tensor], prompt: Sequence[int], n_new: int) -> List[int]:
    toks, out = list(prompt), []
    for _ in range(n_new):
        nxt = int(forward(cfg, p, toks)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out
