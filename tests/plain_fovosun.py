"""A plain, slow Fovosun decoder: whole sequences, no cache, one function a mechanism.

The yardstick of the Fovosun tests.  It shares no code with the package: ``config.json`` as a raw
dict, weights as a ``{name: tensor}`` dict, dense tensor arithmetic on the CPU (float64 unless
told otherwise), every key and every state of a sequence recomputed from its first token.

Notation: T tokens, W the model width, S residual streams, H query heads, G key/value heads, d the
width of one score map's query or key, e the width of a value head, n the taps of a convolution.
"""
from __future__ import annotations

import json
import math
import os
from typing import Callable, Dict, List, Optional

import torch

SWISH_SLOPE = 1.702       # the feed-forward's gate is g * sigmoid(SWISH_SLOPE * g)


def _same(x: torch.Tensor) -> torch.Tensor:
    return x


def store_bf16(x: torch.Tensor) -> torch.Tensor:
    """x rounded to bfloat16 and widened again: what a tensor kept in 16 bits loses.  Handed to the
    functions below as ``store``, it is applied where a 16-bit engine may keep a tensor (the outputs
    of matrix products, of norms, of activations and of the attention), and nowhere in what the
    design computes in 32 bits (scores and softmax, rotations, states, norms' statistics, the
    residual streams): the difference to the exact run shows how far rounding alone moves a result."""
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


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * w


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def rotate_half_split(x: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x [T, heads, d]: the first `dims` elements of every head turn, element i with element
    i + dims/2 by the angle p * base^(-2i/dims); the rest pass."""
    half = dims // 2
    i = torch.arange(half, dtype=x.dtype)
    freq = torch.pow(torch.tensor(base, dtype=x.dtype), -2.0 * i / dims)
    ang = positions.to(x.dtype)[:, None] * freq[None, :]            # [T, half]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def causal_conv(u: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """u [T, C], w [C, n]: y_t = sum_j w[:, j] * u_(t - n + 1 + j), zeros before the first row."""
    T, n = u.shape[0], w.shape[1]
    padded = torch.cat([torch.zeros(n - 1, u.shape[1], dtype=u.dtype), u], dim=0)
    y = torch.zeros_like(u)
    for j in range(n):
        y = y + padded[j:j + T] * w[:, j][None, :]
    return y


def query_temperature(positions: torch.Tensor, coef: float, every: float, dtype) -> torch.Tensor:
    """1 + coef * ln(floor((p + 1) / every) + 1) for every position."""
    return 1.0 + coef * torch.log(torch.floor((positions.to(dtype) + 1.0) / every) + 1.0)


def visible(T: int, window: Optional[int]) -> torch.Tensor:
    """[T, T] bool: key j is seen from i when j <= i and, with a window, i - j < window."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window:
        ok = ok & (i - j < window)
    return ok


def softmax_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, mask: torch.Tensor) -> torch.Tensor:
    """One score map: q [T, H, d], k [T, G, d], v [T, G, e] -> [T, H, e]; head h reads key/value head h // (H / G)."""
    H, G = q.shape[1], k.shape[1]
    rep = H // G
    out = []
    for h in range(H):
        g = h // rep
        s = (q[:, h, :] @ k[:, g, :].T) * scale
        s = s.masked_fill(~mask, float("-inf"))
        out.append(torch.softmax(s, dim=-1) @ v[:, g, :])
    return torch.stack(out, dim=1)


def difference_lambda(w: Dict[str, torch.Tensor], prefix: str, diff: float) -> torch.Tensor:
    return torch.exp((w[prefix + "lq1"] * w[prefix + "lk1"]).sum()) - torch.exp((w[prefix + "lq2"] * w[prefix + "lk2"]).sum()) + diff


def difference_of_maps(a1: torch.Tensor, a2: torch.Tensor, lam, diff: float, eps: float) -> torch.Tensor:
    """a1 - lam * a2, each head divided by its root mean square, times 1 - diff."""
    return unit_rms(a1 - lam * a2, eps) * (1.0 - diff)


# ----------------------------------------------------------------------------
# mixers
# ----------------------------------------------------------------------------
def differential_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, m: dict, eps: float,
                           store: Callable = _same) -> torch.Tensor:
    """Both attention mixers: two score maps over the same values, their outputs subtracted.  What the
    mixer's object names is on (biases when the tensors are there, `conv`, `rot`, `q_temp`, `mask`, a
    gate when the tensor is there), the rest off."""
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)

    def project(name):
        y = h @ w[prefix + name].T
        if prefix + name + ".b" in w:
            y = y + w[prefix + name + ".b"]
        y = store(y)
        if m.get("conv"):
            y = causal_conv(y, w[prefix + name + ".conv"])
        return y

    q = project("q").reshape(T, H, 2, d)
    k = project("k").reshape(T, G, 2, d)
    v = project("v").reshape(T, G, e)
    rot = m.get("rot")
    if rot:
        q = rotate_half_split(q.reshape(T, H * 2, d), pos, rot["base"], rot["dims"]).reshape(T, H, 2, d)
        k = rotate_half_split(k.reshape(T, G * 2, d), pos, rot["base"], rot["dims"]).reshape(T, G, 2, d)
    qt = m.get("q_temp")
    if qt:
        q = q * query_temperature(pos, qt["coef"], qt["every"], h.dtype)[:, None, None, None]
    q, k, v = store(q), store(k), store(v)
    mask = visible(T, (m.get("mask") or {}).get("size"))
    a1 = store(softmax_attention(q[:, :, 0], k[:, :, 0], v, m["scale"], mask))
    a2 = store(softmax_attention(q[:, :, 1], k[:, :, 1], v, m["scale"], mask))
    lam = difference_lambda(w, prefix, m["diff"])
    o = difference_of_maps(a1, a2, lam, m["diff"], eps)              # [T, H, e]
    if prefix + "g" in w:
        o = o * torch.sigmoid(store(h @ w[prefix + "g"].T))[:, :, None]
    o = store(o.reshape(T, H * e))
    return store(o @ w[prefix + "o"].T)


def retention(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, m: dict, eps: float, store: Callable = _same,
              state: Optional[torch.Tensor] = None, first_position: int = 0):
    """Linear attention with one fixed decay per head: S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.
    Returns (output [T, W], the states after the last token [H, d, e])."""
    T = h.shape[0]
    H, d, e = m["heads"], m["dim"], m["vdim"]
    pos = torch.arange(first_position, first_position + T)
    q = store(h @ w[prefix + "q"].T).reshape(T, H, d)
    k = store(h @ w[prefix + "k"].T).reshape(T, H, d)
    v = store(h @ w[prefix + "v"].T).reshape(T, H, e)
    rot = m.get("rot")
    if rot:
        q = rotate_half_split(q, pos, rot["base"], rot["dims"])
        k = rotate_half_split(k, pos, rot["base"], rot["dims"])
    k = k * d ** -0.5
    S = torch.zeros(H, d, e, dtype=h.dtype) if state is None else state.clone()
    decay = torch.tensor(m["decay"], dtype=h.dtype)[:, None, None]
    o = torch.zeros(T, H, e, dtype=h.dtype)
    for t in range(T):
        S = decay * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hde,hd->he", S, q[t])
    o = unit_rms(o, eps).reshape(T, H * e) * silu(store(h @ w[prefix + "g"].T))
    return store(store(o) @ w[prefix + "o"].T), S


# ----------------------------------------------------------------------------
# feed-forwards
# ----------------------------------------------------------------------------
def clamped_glu(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, limit: float, store: Callable = _same) -> torch.Tensor:
    """g = min(gate h, limit), u = clamp(up h, -limit, limit); down(g sigmoid(1.702 g) (u + 1))."""
    g = store(h @ w[prefix + "gate"].T).clamp(max=limit)
    u = store(h @ w[prefix + "up"].T).clamp(min=-limit, max=limit)
    y = store(g * torch.sigmoid(SWISH_SLOPE * g) * (u + 1.0))
    return store(y @ w[prefix + "down"].T)


def router_choice(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, top: int):
    """(experts [T, top], weights [T, top]): the largest logits, softmax over them alone."""
    z = h @ w[prefix + "router"].T + w[prefix + "router.b"]
    val, idx = torch.topk(z, top, dim=-1)
    return idx, torch.softmax(val, dim=-1)


def mixture(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, mlp: dict, store: Callable = _same,
            picks=None) -> torch.Tensor:
    """The routed experts' weighted sum plus the shared expert.  ``picks`` (experts, weights) replaces the
    router's own choice (a test hands in the engine's, so that a close call cannot move a comparison)."""
    idx, wts = picks if picks is not None else router_choice(h, w, prefix, mlp["router"]["top"])
    out = torch.zeros_like(h)
    limit = mlp["expert"]["limit"]
    for e in range(mlp["router"]["experts"]):
        rows, slot = (idx == e).nonzero(as_tuple=True)
        if rows.numel():
            y = clamped_glu(h[rows], w, f"{prefix}e{e}.", limit, store)
            out[rows] = out[rows] + wts[rows, slot].to(h.dtype)[:, None] * y
    if mlp.get("shared"):
        out = out + clamped_glu(h, w, prefix + "shared.", mlp["shared"]["limit"], store)
    return store(out)


def feed_forward(h, w, prefix, mlp, store=_same, picks=None):
    if mlp["kind"] == "dense":
        return clamped_glu(h, w, prefix, mlp["limit"], store)
    return mixture(h, w, prefix, mlp, store, picks)


# ----------------------------------------------------------------------------
# the streams
# ----------------------------------------------------------------------------
def streams_read(xs: torch.Tensor, w_in: torch.Tensor) -> torch.Tensor:
    """xs [S, T, W] -> sum_s in[s] xs[s]."""
    return torch.einsum("s,stw->tw", w_in, xs)


def streams_write(xs: torch.Tensor, y: torch.Tensor, w_mix: torch.Tensor, w_out: torch.Tensor) -> torch.Tensor:
    """new[t] = sum_s mix[s, t] xs[s] + out[t] y, all from the old streams."""
    return torch.einsum("sr,stw->rtw", w_mix, xs) + w_out[:, None, None] * y[None]


# ----------------------------------------------------------------------------
# the model
# ----------------------------------------------------------------------------
def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int], store: Callable = _same, dtype=torch.float64,
            layer_outputs: Optional[list] = None, router_picks=None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence.  ``layer_outputs``: a list that receives the sum of the streams
    after every layer.  ``router_picks``: per routed layer (in order) the (experts, weights) to use."""
    eps = cfg["norm"]["eps"]
    n_streams = cfg.get("streams")
    x = w["embed"][torch.tensor(tokens)].to(dtype) * cfg["embedding"]["scale"]
    xs = x[None].repeat(n_streams, 1, 1) if n_streams else None
    routed = 0
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        for q, sub in ((1, "mix"), (2, "mlp")):
            if sub == "mlp" and layer.get("mlp") is None:
                continue
            inp = streams_read(xs, w[f"{p}hc{q}.in"]) if n_streams else x
            hn = store(rms_norm(inp, w[f"{p}norm{q}"], eps))
            if sub == "mix":
                if layer["type"] == "retention":
                    y, _ = retention(hn, w, p + "mix.", layer["mixer"], eps, store)
                else:
                    y = differential_attention(hn, w, p + "mix.", layer["mixer"], eps, store)
            else:
                picks = None
                if layer["mlp"]["kind"] == "moe":
                    picks = router_picks[routed] if router_picks is not None else None
                    routed += 1
                y = feed_forward(hn, w, p + "mlp.", layer["mlp"], store, picks)
            if n_streams:
                xs = streams_write(xs, y, w[f"{p}hc{q}.mix"], w[f"{p}hc{q}.out"])
            else:
                x = x + y
        if layer_outputs is not None:
            layer_outputs.append(xs.sum(dim=0) if n_streams else x)
    if n_streams:
        x = xs.sum(dim=0)
    hn = store(rms_norm(x, w["final.norm"], eps))
    return hn @ w["head"].T


def generate(cfg: dict, w: Dict[str, torch.Tensor], prompt: List[int], n_new: int) -> List[int]:
    """Greedy continuation: the whole sequence is recomputed for every new token."""
    toks, out = list(prompt), []
    for _ in range(n_new):
        nxt = int(torch.argmax(forward(cfg, w, toks)[-1]))
        toks.append(nxt)
        out.append(nxt)
    return out
