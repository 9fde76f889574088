"""Python faces of the HIP kernels.

Every function checks on the host that shapes, dtypes and devices are what the kernel and its
grid assume, then launches on torch's current stream.  Tensors are only memory here: no torch
arithmetic runs on the product path except the library matrix product in :func:`linear`.
"""
from __future__ import annotations

import collections

from typing import Optional, Tuple

import torch

from . import lib as _lib
from . import profile as _profile

_DT = {torch.float32: 0, torch.bfloat16: 1}

WINDOW_NONE, WINDOW_CHUNK, WINDOW_SLIDING = 0, 1, 2
ACT_SILU, ACT_GELU_TANH, ACT_SWISH_CLAMP = 1, 2, 3      # the gated unit's activation, as the kernels code it
ACTIVATIONS = {"silu": ACT_SILU, "gelu_tanh": ACT_GELU_TANH, "swish_clamp": ACT_SWISH_CLAMP}


def gated_activation(name: str, limit: Optional[float] = None):
    """What the kernels take as ``act`` for the gated unit `name`: its code, or for "swish_clamp" (gate
    g = min(g, limit), up u = clamp(u, -limit, limit), result g sigmoid(1.702 g) (u + 1)) the pair
    (code, limit)."""
    code = ACTIVATIONS[name]
    if code != ACT_SWISH_CLAMP:
        if limit is not None:
            raise ValueError(f"activation {name!r} takes no limit")
        return code
    if limit is None or not float(limit) > 0:
        raise ValueError("the clamped activation needs a positive limit")
    return (code, float(limit))


def _act_pair(act) -> Tuple[int, float]:
    """(code, limit) of an ``act`` argument: a code alone, or a (code, limit) pair."""
    if isinstance(act, tuple):
        return int(act[0]), float(act[1])
    _need(int(act or 0) != ACT_SWISH_CLAMP, "the clamped activation comes with its limit: (code, limit)")
    return int(act or 0), 0.0


class KernelError(RuntimeError):
    pass


def _code(dtype: torch.dtype) -> int:
    try:
        return _DT[dtype]
    except KeyError:
        raise KernelError(f"dtype {dtype} is not taken by the kernels (float32 or bfloat16)") from None


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _dev(*ts) -> None:
    for t in ts:
        if t is not None:
            _need(t.is_cuda, "kernel operands must live on the GPU")
            _need(t.is_contiguous(), "kernel operands must be contiguous")


def _i32(t: Optional[torch.Tensor], name: str) -> None:
    if t is not None:
        _need(t.dtype == torch.int32, f"{name} must be int32")


def _run(name: str, *args) -> None:
    if _profile._active is not None and _profile._active.depth == 0:
        with _profile.section(name[len("sharpi_"):]):       # a launch outside any section: a class of its own
            return _run(name, *args)
    rc = getattr(_lib.load(), name)(*args)
    if rc != 0:
        what = {1001: "a size or option the kernel does not take", 1002: "launch failed"}.get(rc, f"HIP error {rc}")
        raise KernelError(f"{name}: {what}")


# ---------------------------------------------------------------------------
def embed_gather(ids: torch.Tensor, table: torch.Tensor, out: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """out[t] = table[ids[t]] * scale as float32 (the residual stream)."""
    _dev(ids, table, out)
    _i32(ids, "ids")
    _need(ids.dim() == 1 and table.dim() == 2, "embed_gather: ids [T], table [V, H]")
    T, H = ids.shape[0], table.shape[1]
    if out is None:
        out = torch.empty(T, H, dtype=torch.float32, device=table.device)
    _need(out.shape == (T, H) and out.dtype == torch.float32, "embed_gather: out must be float32 [T, H]")
    _run("sharpi_embed_gather", _ptr(ids), _ptr(table), _code(table.dtype), _ptr(out), T, H, float(scale), _stream())
    return out


def scale_softcap(logits: torch.Tensor, scale: float = 1.0, cap: float = 0.0) -> torch.Tensor:
    """logits (float32, contiguous) in place: x * scale, then cap * tanh(x / cap) if cap > 0."""
    _dev(logits)
    _need(logits.dtype == torch.float32 and logits.is_contiguous() and cap >= 0, "scale_softcap: float32 contiguous logits, cap >= 0")
    _run("sharpi_scale_softcap", _ptr(logits), logits.numel(), float(scale), float(cap), _stream())
    return logits


class ExpertSum:
    """A branch output that is still a sum to be formed: row t = sum_j w[t, j] * y[inv_pos[t*k + j]]
    (+ shared[t]); ``weights`` None means ones (scores already applied to the experts' inputs).
    ``add_rmsnorm`` forms it on the fly; ``tensor()`` forms it with a kernel of its own.  Either
    way the sum is rounded once to y's storage type."""

    __slots__ = ("y", "inv_pos", "shared", "n_tokens", "k", "weights")

    def __init__(self, y: torch.Tensor, inv_pos: torch.Tensor, shared: Optional[torch.Tensor], n_tokens: int, k: int,
                 weights: Optional[torch.Tensor] = None):
        _need(y.dim() == 2 and inv_pos.numel() == n_tokens * k, "ExpertSum: y [rows, H], inv_pos [T*k]")
        if shared is not None:
            _need(shared.shape == (n_tokens, y.shape[1]) and shared.dtype == y.dtype and shared.is_contiguous(),
                  "ExpertSum: shared must be contiguous [T, H] of y's dtype")
        if weights is not None:
            _need(weights.numel() == n_tokens * k and weights.dtype == torch.float32 and weights.is_contiguous(),
                  "ExpertSum: weights must be contiguous float32 [T, k]")
        self.y, self.inv_pos, self.shared, self.n_tokens, self.k, self.weights = y, inv_pos, shared, n_tokens, k, weights

    @property
    def shape(self):
        return (self.n_tokens, self.y.shape[1])

    @property
    def dtype(self):
        return self.y.dtype

    def tensor(self) -> torch.Tensor:
        return moe_combine(self.y[: self.n_tokens * self.k], self.inv_pos, self.shared, self.n_tokens, self.k,
                           self.weights)


def add_rmsnorm(h: torch.Tensor, delta, weight: Optional[torch.Tensor], eps: float,
                out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None, write_back: bool = True,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """(h + delta) -> RMSNorm -> out; the sum goes back into h unless rows are gathered.
    delta: a tensor, an ExpertSum, or None."""
    lazy = delta if isinstance(delta, ExpertSum) else None
    if lazy is not None and h.shape[1] % 8 != 0:
        delta, lazy = lazy.tensor(), None          # the kernel folds a sum in only at widths that are multiples of 8
    base = lazy.y if lazy is not None else delta
    _dev(h, base, weight, rows, out, lazy.weights if lazy is not None else None)
    _i32(rows, "rows")
    _need(h.dim() == 2 and h.dtype == torch.float32, "add_rmsnorm: h must be float32 [T, H]")
    T, H = h.shape
    if delta is not None:
        _need(tuple(delta.shape) == tuple(h.shape), f"add_rmsnorm: delta {tuple(delta.shape)} vs h {tuple(h.shape)}")
    if weight is not None:
        _need(weight.shape == (H,), f"add_rmsnorm: weight {tuple(weight.shape)} vs width {H}")
    n_out = T if rows is None else rows.shape[0]
    if rows is not None:
        write_back = False
    if out is None:
        out = torch.empty(n_out, H, dtype=out_dtype, device=h.device)
    _need(out.shape == (n_out, H) and out.dtype == out_dtype, "add_rmsnorm: out has the wrong shape or dtype")
    _run("sharpi_add_rmsnorm", _ptr(h), _ptr(base), _code(base.dtype) if base is not None else 0,
         _ptr(weight), _code(weight.dtype) if weight is not None else 0, _ptr(out), _code(out_dtype), _ptr(rows),
         n_out, H, float(eps), 1 if write_back else 0,
         _ptr(lazy.inv_pos) if lazy is not None else None, _ptr(lazy.shared) if lazy is not None else None,
         _ptr(lazy.weights) if lazy is not None else None, lazy.k if lazy is not None else 0, _stream())
    return out


def gated_act(gate_up: torch.Tensor, scale: Optional[torch.Tensor] = None, act=ACT_SILU,
              bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """[M, 2I] (gate columns, then up columns) -> act(s*g) * (s*u) [M, I]; act: ACT_SILU,
    ACT_GELU_TANH, or (ACT_SWISH_CLAMP, limit) (see :func:`gated_activation`).  ``bias`` (float32 [2I])
    is added to the gate and up columns first, in float."""
    _dev(gate_up, scale, bias)
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (gate_up.shape[1],), "gated_act: bias must be float32 [2I]")
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0, "gated_act: input must be [M, 2I]")
    M, I2 = gate_up.shape
    if scale is not None:
        _need(scale.dtype == torch.float32 and scale.shape == (M,), "gated_act: scale must be float32 [M]")
    out = torch.empty(M, I2 // 2, dtype=gate_up.dtype, device=gate_up.device)
    _run("sharpi_silu_mul", _ptr(gate_up), _ptr(scale), _ptr(out), _code(gate_up.dtype), M, I2 // 2, *_act_pair(act), _ptr(bias), _stream())
    return out


def silu_mul(gate_up: torch.Tensor, scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """[M, 2I] (gate columns, then up columns) -> silu(s*g) * (s*u) [M, I]."""
    return gated_act(gate_up, scale, ACT_SILU)


def moe_combine(y: torch.Tensor, inv_pos: torch.Tensor, shared: Optional[torch.Tensor], n_tokens: int,
                k: int, weights: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t] = sum_j w[t, j] * y[inv_pos[t*k+j]] (+ shared[t]); weights None: ones."""
    _dev(y, inv_pos, shared, weights)
    _i32(inv_pos, "inv_pos")
    _need(y.dim() == 2 and y.shape[0] == n_tokens * k and inv_pos.numel() == n_tokens * k,
          "moe_combine: y must be [T*k, H] and inv_pos [T*k]")
    H = y.shape[1]
    if shared is not None:
        _need(shared.shape == (n_tokens, H) and shared.dtype == y.dtype, "moe_combine: shared must be [T, H]")
    if weights is not None:
        _need(weights.numel() == n_tokens * k and weights.dtype == torch.float32, "moe_combine: weights must be float32 [T, k]")
    out = torch.empty(n_tokens, H, dtype=y.dtype, device=y.device)
    _run("sharpi_moe_combine", _ptr(y), _ptr(inv_pos), _ptr(shared), _ptr(weights), _ptr(out), _code(y.dtype), n_tokens,
         H, k, _stream())
    return out


def add_bias(x: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """x [T, N] += bias [N] (float32), in place: the sum in float, rounded to x's storage."""
    _dev(x, bias)
    _need(x.dim() == 2 and x.is_contiguous() and bias.dtype == torch.float32 and bias.shape == (x.shape[1],)
          and bias.is_contiguous(), "add_bias: x [T, N] contiguous and bias float32 [N] wanted")
    _run("sharpi_add_bias", _ptr(x), _code(x.dtype), _ptr(bias), x.shape[0], x.shape[1], _stream())
    return x


def cast(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    _dev(x)
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    _run("sharpi_cast", _ptr(x), _code(x.dtype), _ptr(out), _code(dtype), x.numel(), _stream())
    return out


def random_fill(out: torch.Tensor, key: int, kind: int, std: float = 0.02, lo: float = 0.9, hi: float = 1.1) -> torch.Tensor:
    """Fill `out` (float32, bfloat16, or int32 for integers) with the seeded values of
    weights/random_fill.py: element i is a function of (key, i) alone, the same bits as the host makes."""
    from ..weights import random_fill as rf

    _dev(out)
    if kind == rf.FILL_INT:
        _need(out.dtype == torch.int32, "random_fill: integers go into int32")
        code = 0
    else:
        code = _code(out.dtype)
    lo_f, span_f = rf.uniform_fixed(lo, hi)
    _run("sharpi_random_fill", _ptr(out), code, out.numel(), int(key) & ((1 << 64) - 1), int(kind),
         rf.normal_scale(std), lo_f, span_f, _stream())
    return out


# ---------------------------------------------------------------------------
def _cache_shapes_ok(k_cache: torch.Tensor, v_cache: torch.Tensor, nkv: int, hd: int, vd: Optional[int] = None) -> bool:
    """K [pages, nkv, page_size, hd] and V [pages, nkv, vd, page_size] (vd: the values' width, hd unless given)."""
    return (k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.shape[1] == nkv and k_cache.shape[3] == hd
            and v_cache.shape == (k_cache.shape[0], nkv, vd or hd, k_cache.shape[2]))


PAIRS_INTERLEAVED, PAIRS_HALF_SPLIT = 0, 1


def rope_kv(qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, slot_mapping: torch.Tensor,
            positions: torch.Tensor, inv_freq: Optional[torch.Tensor], qk_norm: bool, eps: float,
            temperature: Optional[Tuple[float, float]], nh: int, nkv: int, hd: int,
            pair_layout: int = PAIRS_INTERLEAVED, bias: Optional[torch.Tensor] = None, vd: Optional[int] = None,
            extra_columns: int = 0) -> torch.Tensor:
    """Rotate / norm / scale the heads of qkv [T, (nh+nkv)*hd + nkv*vd] (vd, the values' width, is hd
    unless given); K and V go into the layer's
    cache [pages, nkv, page_size, hd] at slot_mapping; returns q [T, nh*hd].  inv_freq [r/2]
    rotates the first r <= hd elements of every head, in pairs (2i, 2i+1) or (i, i + r/2)
    (``pair_layout``); the rest of the head passes through.  ``bias`` (float32, one value per
    column of q, k and v) is added to every row first, in float.  ``extra_columns``: further columns of
    each row behind q, k and v (another product's outputs made by the same launch), which are left alone."""
    _dev(qkv, k_cache, v_cache, slot_mapping, positions, inv_freq, bias)
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (qkv.shape[1] - extra_columns,) and bias.is_contiguous(),
              "rope_kv: bias must be float32, one value per column of qkv")
    _i32(slot_mapping, "slot_mapping")
    _i32(positions, "positions")
    T = qkv.shape[0]
    vd = int(vd or hd)
    _need(qkv.dim() == 2 and extra_columns >= 0 and qkv.shape[1] == (nh + nkv) * hd + nkv * vd + extra_columns,
          "rope_kv: qkv must be [T, (nh+nkv)*hd + nkv*vd (+ extra_columns)]")
    _need(_cache_shapes_ok(k_cache, v_cache, nkv, hd, vd), "rope_kv: caches must be K [pages, nkv, page_size, hd], V [pages, nkv, vd, page_size]")
    _need(k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype, "rope_kv: cache dtype differs from qkv's")
    _need(slot_mapping.shape == (T,) and positions.shape == (T,), "rope_kv: slot_mapping / positions must be [T]")
    rotary_dim = 0
    if inv_freq is not None:
        _need(inv_freq.dtype == torch.float32 and inv_freq.dim() == 1 and 1 <= inv_freq.shape[0] <= hd // 2,
              "rope_kv: inv_freq must be float32 [rotary_dim / 2], rotary_dim <= hd")
        rotary_dim = 2 * inv_freq.shape[0]
    _need(pair_layout in (PAIRS_INTERLEAVED, PAIRS_HALF_SPLIT), "rope_kv: pair_layout must be interleaved (0) or half-split (1)")
    page_size = k_cache.shape[2]
    q_out = torch.empty(T, nh * hd, dtype=qkv.dtype, device=qkv.device)
    fs, asc = temperature if temperature is not None else (1.0, 0.0)
    _run("sharpi_rope_kv", _ptr(qkv), _ptr(q_out), _ptr(k_cache), _ptr(v_cache), _code(qkv.dtype),
         _ptr(slot_mapping), _ptr(positions), _ptr(inv_freq), _ptr(bias), 1 if qk_norm else 0, float(eps),
         1 if temperature is not None else 0, float(fs), float(asc), T, nh, nkv, hd, vd, page_size, int(pair_layout),
         rotary_dim, qkv.shape[1], _stream())
    return q_out


def _sink_args(sink, nh: int):
    """The two arguments the attention kernels take for a sink: (flag, values).  ``sink`` False / None: no
    sink; True: one more term exp(0) in the denominator; a float32 tensor [nh]: exp(sink[head]), a
    learned score per head (not scaled, without a value)."""
    if sink is None or sink is False:
        return 0, None
    if sink is True:
        return 1, None
    _dev(sink)
    _need(sink.dtype == torch.float32 and sink.shape == (nh,), "attention: a learned sink must be float32 [nh]")
    return 1, _ptr(sink)


def attention_generic(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                      entry_of_token: torch.Tensor, positions: torch.Tensor, window_kind: int, window: int,
                      scale: float, nh: int, nkv: int, hd: int, vd: Optional[int] = None, softcap: float = 0.0,
                      sink: bool = False) -> torch.Tensor:
    """Attention of every token of the batch over its request's pages; float arithmetic.  Values
    (and so the output, [T, nh*vd]) may have another width than keys.  softcap > 0: scores become
    softcap * tanh(score / softcap); sink: one more term exp(0), without a value, in the softmax's
    denominator."""
    _dev(q, k_cache, v_cache, block_table, entry_of_token, positions)
    _i32(block_table, "block_table")
    _i32(entry_of_token, "entry_of_token")
    _i32(positions, "positions")
    T = q.shape[0]
    vd = int(vd or hd)
    _need(q.shape == (T, nh * hd), "attention: q must be [T, nh*hd]")
    _need(_cache_shapes_ok(k_cache, v_cache, nkv, hd, vd) and k_cache.dtype == q.dtype and v_cache.dtype == q.dtype,
          "attention: caches must be K [pages, nkv, page_size, hd], V [pages, nkv, vd, page_size] of q's dtype")
    _need(block_table.dim() == 2, "attention: block_table must be [entries, max_blocks]")
    _need(entry_of_token.shape == (T,) and positions.shape == (T,), "attention: per-token arrays must be [T]")
    out = torch.empty(T, nh * vd, dtype=q.dtype, device=q.device)
    _run("sharpi_attention_generic", _ptr(q), _ptr(k_cache), _ptr(v_cache), _code(q.dtype), _ptr(block_table),
         _ptr(entry_of_token), _ptr(positions), _ptr(out), int(window_kind), int(window), float(scale), T, nh, nkv,
         hd, vd, k_cache.shape[2], block_table.shape[1], k_cache.shape[0], float(softcap), *_sink_args(sink, nh), _stream())
    return out


DECODE_RUN_KEYS = _lib.DECODE_RUN_KEYS   # keys per block of the decode kernel (fixed: sums must not depend on the batch)


def decode_max_splits(max_context: int) -> int:
    """Runs of DECODE_RUN_KEYS keys that cover every token of a context of `max_context` tokens,
    whatever its window: runs are aligned to absolute positions, so a token at position p whose
    first visible key is s takes ((p >> 4) - (s >> 4)) // 16 + 1 of them, most for s = 0."""
    return ((max(1, int(max_context)) - 1) >> 4) // (DECODE_RUN_KEYS // 16) + 1


def decode_attention_ok(dtype: torch.dtype, hd: int) -> bool:
    return dtype == torch.bfloat16 and _lib.attention_takes("decode", hd)


def attention_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                     entry_of_token: torch.Tensor, positions: torch.Tensor, token_list: Optional[torch.Tensor],
                     max_context: int, window_kind: int, window: int, scale: float, nh: int, nkv: int, hd: int,
                     out: Optional[torch.Tensor] = None, softcap: float = 0.0, sink: bool = False) -> torch.Tensor:
    """Split-K flash-decode for the listed tokens (all tokens if token_list is None), each a
    single query over its request's pages.  `max_context` bounds position + 1 of every token."""
    _dev(q, k_cache, v_cache, block_table, entry_of_token, positions, token_list, out)
    _i32(block_table, "block_table")
    _i32(entry_of_token, "entry_of_token")
    _i32(positions, "positions")
    _i32(token_list, "token_list")
    T = q.shape[0]
    _need(q.shape == (T, nh * hd) and decode_attention_ok(q.dtype, hd), "attention_decode: q must be bfloat16 [T, nh*hd], hd a head size the kernel is compiled for")
    _need(_cache_shapes_ok(k_cache, v_cache, nkv, hd) and k_cache.dtype == q.dtype and v_cache.dtype == q.dtype,
          "attention_decode: caches must be K [pages, nkv, page_size, hd], V [pages, nkv, hd, page_size] bfloat16")
    _need(block_table.dim() == 2 and entry_of_token.shape == (T,) and positions.shape == (T,),
          "attention_decode: block_table [entries, max_blocks], per-token arrays [T]")
    n_list = T if token_list is None else token_list.shape[0]
    if out is None:
        out = torch.empty_like(q)
    _need(out.shape == q.shape and out.dtype == q.dtype, "attention_decode: out must match q")
    max_splits = decode_max_splits(max_context)
    part_o = torch.empty(n_list * nh * max_splits * hd, dtype=torch.float32, device=q.device)
    part_ml = torch.empty(n_list * nh * max_splits * 2, dtype=torch.float32, device=q.device)
    _run("sharpi_attention_decode", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), _ptr(entry_of_token),
         _ptr(positions), _ptr(token_list), _ptr(part_o), _ptr(part_ml), _ptr(out), int(window_kind), int(window),
         float(scale), n_list, nh, nkv, hd, k_cache.shape[2], block_table.shape[1], k_cache.shape[0], max_splits,
         float(softcap), *_sink_args(sink, nh), _stream())
    return out


PREFILL_TILE_TOKENS = _lib.PREFILL_TILE_TOKENS   # tokens per block of the prefill kernel (32 per wave)


def prefill_attention_ok(dtype: torch.dtype, hd: int) -> bool:
    return dtype == torch.bfloat16 and _lib.attention_takes("prefill", hd)


def attention_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                      positions: torch.Tensor, tiles: torch.Tensor, window_kind: int, window: int, scale: float,
                      nh: int, nkv: int, hd: int, out: Optional[torch.Tensor] = None,
                      tile_tokens: int = PREFILL_TILE_TOKENS, softcap: float = 0.0, sink: bool = False) -> torch.Tensor:
    """Flash attention for the listed tiles: tiles int32 [n, 3] = (entry, first token, rows <=
    tile_tokens), the tokens of a tile consecutive in one entry.  tile_tokens (128, or 64: blocks of
    half the rows, for short prompts) is what the caller cut the tiles to; a row's result does not
    depend on it."""
    _dev(q, k_cache, v_cache, block_table, positions, tiles, out)
    _i32(block_table, "block_table")
    _i32(positions, "positions")
    _i32(tiles, "tiles")
    T = q.shape[0]
    _need(q.shape == (T, nh * hd) and prefill_attention_ok(q.dtype, hd),
          "attention_prefill: q must be bfloat16 [T, nh*hd], hd a head size the kernel is compiled for")
    _need(_cache_shapes_ok(k_cache, v_cache, nkv, hd) and k_cache.dtype == q.dtype and v_cache.dtype == q.dtype,
          "attention_prefill: caches must be K [pages, nkv, page_size, hd], V [pages, nkv, hd, page_size] bfloat16")
    _need(block_table.dim() == 2 and positions.shape == (T,) and tiles.dim() == 2 and tiles.shape[1] == 3,
          "attention_prefill: block_table [entries, max_blocks], positions [T], tiles [n, 3]")
    if out is None:
        out = torch.empty_like(q)
    _need(out.shape == q.shape and out.dtype == q.dtype, "attention_prefill: out must match q")
    _run("sharpi_attention_prefill", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), _ptr(positions),
         _ptr(tiles), _ptr(out), tiles.shape[0], int(tile_tokens), int(window_kind), int(window), float(scale), nh,
         nkv, hd, k_cache.shape[2], block_table.shape[1], k_cache.shape[0], float(softcap), *_sink_args(sink, nh), _stream())
    return out


# ---------------------------------------------------------------------------
def gemm_tiled(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """x [M, K] @ w [N, K]^T with float FMA chains (batch-invariant)."""
    _dev(x, w)
    _need(x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1], f"gemm: x {tuple(x.shape)} vs w {tuple(w.shape)}")
    _need(x.dtype == w.dtype, "gemm: x and w must share a dtype")
    out_dtype = out_dtype or x.dtype
    M, K = x.shape
    N = w.shape[0]
    out = torch.empty(M, N, dtype=out_dtype, device=x.device)
    _run("sharpi_gemm_tiled", _ptr(x), _ptr(w), _ptr(out), _code(x.dtype), _code(out_dtype), M, N, K, None, None, 0,
         _stream())
    return out


# ---------------------------------------------------------------------------
# layers whose norms sit on the branch outputs; latent attention
# ---------------------------------------------------------------------------
def norm_add(h: torch.Tensor, delta, weight: torch.Tensor, eps: float,
             out_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """h += unit_rms(delta) * weight, in place in float; with ``out_dtype`` the new h is also
    returned in that storage type (what the next branch reads).  delta: a tensor [T, H] or an
    ExpertSum without a shared part (formed on the fly, rounded once to its storage type)."""
    lazy = delta if isinstance(delta, ExpertSum) else None
    if lazy is not None and lazy.shared is not None:
        delta, lazy = lazy.tensor(), None
    base = lazy.y if lazy is not None else delta
    _dev(h, base, weight, lazy.weights if lazy is not None else None)
    _need(h.dim() == 2 and h.dtype == torch.float32, "norm_add: h must be float32 [T, H]")
    T, H = h.shape
    _need(tuple(delta.shape) == (T, H), f"norm_add: delta {tuple(delta.shape)} vs h {tuple(h.shape)}")
    _need(weight.dtype == torch.float32 and weight.shape == (H,), "norm_add: weight must be float32 [H]")
    if lazy is not None:
        _need(base.dim() == 2 and base.shape[1] == H, "norm_add: the experts' rows must be [rows, H]")
    out = torch.empty(T, H, dtype=out_dtype, device=h.device) if out_dtype is not None else None
    _run("sharpi_norm_add", _ptr(h), _ptr(base), _code(base.dtype), _ptr(weight), _ptr(out),
         _code(out_dtype) if out_dtype is not None else 0, T, H, float(eps),
         _ptr(lazy.inv_pos) if lazy is not None else None, _ptr(lazy.weights) if lazy is not None else None,
         lazy.k if lazy is not None else 0, _stream())
    return out


def latent_prep(proj: torch.Tensor, q_off: int, kv_off: Optional[int], q_full: torch.Tensor,
                rows: Optional[torch.Tensor], slot_mapping: Optional[torch.Tensor], positions: torch.Tensor,
                inv_freq: Optional[torch.Tensor], norm_w: Optional[torch.Tensor], eps: float, nh: int, dn: int, dr: int,
                rank: int) -> None:
    """Per token of proj [T, ld] (queries [nh, dn + dr] at column q_off, the down projection
    [rank + dr] at column kv_off, None: this layer makes no latent): the rotated query parts go to
    columns rank.. of every head of q_full [T, nh, rank + dr]; the latent rms_norm(first rank
    elements) * norm_w and the rotated key part go side by side into the cache rows
    [pages, 1, page_size, rank + dr] at slot_mapping (-1: nothing stored).  inv_freq float32
    [pairs]: pairs (2i, 2i + 1) of the rotated parts turn by position * inv_freq[i]."""
    _dev(proj, q_full, rows, slot_mapping, positions, inv_freq, norm_w)
    _i32(slot_mapping, "slot_mapping")
    _i32(positions, "positions")
    T, ld = proj.shape
    D = rank + dr
    _need(q_full.shape == (T, nh * D) and q_full.dtype == proj.dtype, "latent_prep: q_full must be [T, nh * (rank + dr)] of proj's dtype")
    _need(positions.shape == (T,), "latent_prep: positions must be [T]")
    n_pairs = 0
    if inv_freq is not None:
        _need(inv_freq.dtype == torch.float32 and inv_freq.dim() == 1 and 2 * inv_freq.shape[0] <= dr,
              "latent_prep: inv_freq must be float32 [pairs], 2 * pairs <= dr")
        n_pairs = inv_freq.shape[0]
    if kv_off is not None:
        _need(rows is not None and rows.dim() == 4 and rows.shape[1] == 1 and rows.shape[3] == D and rows.dtype == proj.dtype,
              "latent_prep: cache rows must be [pages, 1, page_size, rank + dr] of proj's dtype")
        _need(slot_mapping is not None and slot_mapping.shape == (T,), "latent_prep: slot_mapping must be [T]")
        _need(norm_w is not None and norm_w.dtype == torch.float32 and norm_w.shape == (rank,), "latent_prep: norm_w must be float32 [rank]")
    _run("sharpi_latent_prep", _ptr(proj), _code(proj.dtype), ld, int(q_off), -1 if kv_off is None else int(kv_off),
         _ptr(q_full), _ptr(rows) if kv_off is not None else None, _ptr(slot_mapping) if kv_off is not None else None,
         _ptr(positions), _ptr(inv_freq), n_pairs, _ptr(norm_w) if kv_off is not None else None, float(eps), T, nh, dn, dr,
         rank, _stream())


def head_gemm(x: torch.Tensor, x_off: int, sx: int, w: torch.Tensor, out: torch.Tensor, out_off: int, so: int,
              gate: Optional[torch.Tensor] = None, gate_off: int = 0) -> torch.Tensor:
    """One product per head: out[t, out_off + h * so + n] = sum_k x[t, x_off + h * sx + k] * w[h, n, k]
    for w [nh, N, K], times sigmoid(gate[t, gate_off + h * N + n]) where a gate is given.  x, out and
    gate are rows of one storage type; every sum is one float chain in ascending k."""
    _dev(x, w, out, gate)
    _need(x.dim() == 2 and out.dim() == 2 and w.dim() == 3 and x.shape[0] == out.shape[0], "head_gemm: x [T, ..], out [T, ..], w [nh, N, K]")
    nh, N, K = w.shape
    _need(x.dtype == w.dtype == out.dtype and (gate is None or gate.dtype == x.dtype), "head_gemm: one storage type for all operands")
    ldx, ldo = x.shape[1], out.shape[1]
    _need(x_off >= 0 and sx >= K and x_off + (nh - 1) * sx + K <= ldx, "head_gemm: the heads' inputs do not fit x")
    _need(out_off >= 0 and so >= N and out_off + (nh - 1) * so + N <= ldo, "head_gemm: the heads' outputs do not fit out")
    width = x.element_size()
    gp, ldg = None, 0
    if gate is not None:
        _need(gate.dim() == 2 and gate.shape[0] == x.shape[0] and gate_off >= 0 and gate_off + nh * N <= gate.shape[1],
              "head_gemm: the gate does not fit")
        gp, ldg = gate.data_ptr() + gate_off * width, gate.shape[1]
    _run("sharpi_head_gemm", x.data_ptr() + x_off * width, _code(x.dtype), ldx, sx, _ptr(w),
         out.data_ptr() + out_off * width, ldo, so, gp, ldg, x.shape[0], nh, N, K, _stream())
    return out


LATENT_MAX_RANK = 512    # the latent attention kernels hold this many value elements a row


LATENT_DECODE_RUN_KEYS = 128     # keys a block of the matrix-core latent kernel walks in steps of single tokens
LATENT_PROMPT_RUN_KEYS = 1024    # ... at least, in steps with prompt portions (at most two runs a row)


def latent_run_keys(max_context: int, prompt_step: bool) -> int:
    """Keys per run of the matrix-core latent attention kernel.  Runs start at multiples of this,
    whatever the batch.  Steps of single tokens take short runs (many blocks for few rows); steps
    with prompt portions take runs of at least half the longest context, so that a row has at most
    two and the scratch for unmerged runs stays small."""
    if not prompt_step:
        return LATENT_DECODE_RUN_KEYS
    run = LATENT_PROMPT_RUN_KEYS
    while 2 * run < max_context:
        run *= 2
    return run


def latent_mfma_ok(dtype: torch.dtype, rank: int, dr: int, window_kind: int = WINDOW_NONE) -> bool:
    return dtype == torch.bfloat16 and window_kind == WINDOW_NONE and _lib.latent_attention_takes(rank, dr)


def attention_latent(q: torch.Tensor, rows: torch.Tensor, group, ctx, scale: float, nh: int, rank: int, dr: int,
                     sink: Optional[torch.Tensor] = None, window_kind: int = WINDOW_NONE, window: int = 0,
                     kernel: Optional[str] = None) -> torch.Tensor:
    """Attention of nh query heads over one shared cache row per key (rows [pages, 1, page_size,
    rank + dr]): score = scale * q . row over all rank + dr elements, value = the row's first rank
    elements, softmax in float with exp(sink[h]) as one more term of the denominator where sinks
    (float32 [nh]) are given.  q [T, nh * (rank + dr)] -> [T, nh * rank].  bfloat16 rows of sizes
    the matrix-core kernel takes go there (prompt tiles and single tokens from the step's work
    lists, runs merged afterwards); everything else, and ``kernel="generic"``, through the float kernel."""
    _dev(q, rows, group.block_table, ctx.entry_of_token, ctx.positions, sink)
    T = q.shape[0]
    D = rank + dr
    _need(q.shape == (T, nh * D), "attention_latent: q must be [T, nh * (rank + dr)]")
    _need(rows.dim() == 4 and rows.shape[1] == 1 and rows.shape[3] == D and rows.dtype == q.dtype,
          "attention_latent: cache rows must be [pages, 1, page_size, rank + dr] of q's dtype")
    _need(1 <= rank <= LATENT_MAX_RANK, f"attention_latent: a latent of {rank} is not taken (1 to {LATENT_MAX_RANK})")
    if sink is not None:
        _need(sink.dtype == torch.float32 and sink.shape == (nh,), "attention_latent: sink must be float32 [nh]")
    _i32(group.block_table, "block_table")
    _need(group.block_table.dim() == 2 and ctx.entry_of_token.shape == (T,) and ctx.positions.shape == (T,),
          "attention_latent: block_table [entries, max_blocks], per-token arrays [T]")
    out = torch.empty(T, nh * rank, dtype=q.dtype, device=q.device)
    mfma = latent_mfma_ok(q.dtype, rank, dr, window_kind) and (ctx.n_decode or ctx.n_prefill_tiles) and group.max_context > 0
    _need(kernel in (None, "generic", "mfma") and (kernel != "mfma" or mfma), "attention_latent: this step cannot take the kernel asked for")
    if mfma and kernel != "generic":
        run = latent_run_keys(group.max_context, bool(ctx.n_prefill_tiles))
        max_runs = (group.max_context + run - 1) // run
        part_o = part_ml = None
        if max_runs > 1:
            part_o = torch.empty(T * nh * max_runs * rank, dtype=torch.float32, device=q.device)
            part_ml = torch.empty(T * nh * max_runs * 2, dtype=torch.float32, device=q.device)
        common = (_ptr(sink), _ptr(out), _ptr(part_o), _ptr(part_ml), float(scale), nh, rank, dr, run, max_runs,
                  rows.shape[2], group.block_table.shape[1], rows.shape[0], _stream())
        if ctx.n_prefill_tiles:
            _i32(ctx.prefill_tiles, "tiles")
            _need(ctx.prefill_tiles.dim() == 2 and ctx.prefill_tiles.shape[1] == 3, "attention_latent: tiles [n, 3]")
            _run("sharpi_attention_latent_mfma", _ptr(q), _ptr(rows), _ptr(group.block_table), _ptr(ctx.entry_of_token),
                 _ptr(ctx.positions), _ptr(ctx.prefill_tiles), None, ctx.prefill_tiles.shape[0], int(ctx.prefill_tile_tokens), *common)
        if ctx.n_decode:
            _i32(ctx.decode_tokens, "decode_tokens")
            _run("sharpi_attention_latent_mfma", _ptr(q), _ptr(rows), _ptr(group.block_table), _ptr(ctx.entry_of_token),
                 _ptr(ctx.positions), None, _ptr(ctx.decode_tokens), int(ctx.n_decode), 0, *common)
        if max_runs > 1:
            _run("sharpi_attention_latent_merge", _ptr(part_o), _ptr(part_ml), _ptr(ctx.positions), None, T, _ptr(sink),
                 _ptr(out), nh, rank, run, max_runs, _stream())
        return out
    _run("sharpi_attention_latent", _ptr(q), _ptr(rows), _code(q.dtype), _ptr(group.block_table), _ptr(ctx.entry_of_token),
         _ptr(ctx.positions), _ptr(sink), _ptr(out), int(window_kind), int(window), float(scale), T, nh, rank, dr,
         rows.shape[2], group.block_table.shape[1], rows.shape[0], _stream())
    return out


# ---------------------------------------------------------------------------
# weights stored for streaming
# ---------------------------------------------------------------------------
class PackedWeight:
    """A bfloat16 matrix [N, K] (or a stack [E, N, K]) stored tile by tile for the decode kernels:
    [N/16][K/128][16 runs of 8 k][16 rows][8], the 4 KB of a (16-row tile, 128-wide unit) in the
    order a wave's lanes read them, so that a wave's load is one contiguous kilobyte.  ``packed``
    has the logical shape but that element order; ``rows`` is the ordinary row-major matrix, kept
    where the library's product (which wants rows) also multiplies by it, else None."""

    __slots__ = ("packed", "rows", "shape", "dtype")

    def __init__(self, packed: torch.Tensor, rows: Optional[torch.Tensor]):
        self.packed, self.rows = packed, rows
        self.shape, self.dtype = packed.shape, packed.dtype

    def dim(self) -> int:
        return len(self.shape)

    def select(self, e: int) -> "PackedWeight":
        """Matrix e of a stack (a view)."""
        return PackedWeight(self.packed[e], self.rows[e] if self.rows is not None else None)


def can_pack(w: torch.Tensor) -> bool:
    return w.dtype == torch.bfloat16 and w.dim() in (2, 3) and w.shape[-2] % 16 == 0 and w.shape[-1] % 128 == 0


def pack_into(dst: torch.Tensor, w: torch.Tensor) -> None:
    """Write w [.., N, K] into dst (same shape, contiguous) in packed order."""
    _need(dst.shape == w.shape and dst.is_contiguous() and can_pack(w), "pack_into: shapes must match and be packable")
    N, K = w.shape[-2], w.shape[-1]
    lead = w.shape[:-2]
    src = w.reshape(*lead, N // 16, 16, K // 128, 16, 8)
    n = len(lead)
    dst.view(*lead, N // 16, K // 128, 16, 16, 8).copy_(src.permute(*range(n), n, n + 2, n + 3, n + 1, n + 4))


_KEEP_ROWS = True


def keep_row_major_copies(keep: bool) -> None:
    """Whether matrices that are packed for the decode kernels also keep their row-major copy for
    the library's product at prompt size (faster prefill, about a tenth more weight memory), or
    only the packed copy (every product then runs in this library's kernels).  Read when weights
    are loaded."""
    global _KEEP_ROWS
    _KEEP_ROWS = bool(keep)


def pack_weight(w: torch.Tensor, keep_rows: Optional[bool] = None):
    """w as a PackedWeight if its shape and type allow it, else w itself."""
    if keep_rows is None:
        keep_rows = _KEEP_ROWS
    if not can_pack(w):
        return w
    packed = torch.empty_like(w, memory_format=torch.contiguous_format)
    pack_into(packed, w)
    return PackedWeight(packed, w if keep_rows else None)


def unpack_weight(w: "PackedWeight") -> torch.Tensor:
    """The row-major matrix of a PackedWeight (a copy unless it is kept)."""
    if w.rows is not None:
        return w.rows
    N, K = w.shape[-2], w.shape[-1]
    lead = tuple(w.shape[:-2])
    n = len(lead)
    src = w.packed.view(*lead, N // 16, K // 128, 16, 16, 8)
    return src.permute(*range(n), n, n + 3, n + 1, n + 2, n + 4).reshape(*lead, N, K).contiguous()


def _unwrap(w):
    """(tensor in the kernel's order, packed?) of a weight given as a tensor or a PackedWeight."""
    return (w.packed, True) if isinstance(w, PackedWeight) else (w, False)


# ---------------------------------------------------------------------------
# the weight-streaming product for few rows (decode)
# ---------------------------------------------------------------------------
SKINNY_MAX_ROWS = 64          # rows the kernel multiplies against one stream of a weight tile (4 blocks of 16)
SKINNY_MAX_ROWS_PLAIN = 32    # plain form: beyond two row blocks the library's product is faster (measured at the
SKINNY_MAX_ROWS_TALL = 32     # model's projection shapes: 18 against 23 us at 32 rows, 28 against 23.5 at 64)
SKINNY_TALL = 65536


def skinny_ok(M: int, N: int, K: int, grouped: bool = False) -> bool:
    limit = SKINNY_MAX_ROWS if grouped else SKINNY_MAX_ROWS_TALL if N >= SKINNY_TALL else SKINNY_MAX_ROWS_PLAIN
    return 0 < M <= limit and K % 128 == 0 and N % 4 == 0


def skinny_plan(N: int, K: int, row_blocks: int = 1, groups: int = 1, act: bool = False):
    """(R, NW): 16-row weight tiles per block and waves per block splitting K (measured on
    MI355X over the projection shapes of the model).  NW, which decides the order of a row's
    sums, depends on nothing (so a row's result does not change with the batch); R only says how
    many independent columns a block computes: two tiles where a block holds one block of 16
    rows (the kernel then keeps two K units in flight per wave), four for wide matrices with
    more rows; one where two would make between one and two blocks per compute unit (some
    units would then stream twice what the others do: 30.7 against 33.3 us for the merged down
    projection of one token)."""
    if row_blocks > 1:
        return (4 if N >= 12288 else 2), 8
    blocks = groups * ((N + 31) // 32)
    units = compute_units()
    return (1 if not act and units < blocks < 2 * units else 2), 8


_COMPUTE_UNITS: dict = {}


def compute_units(device=None) -> int:
    """Compute units of the GPU the launches are laid out for: asked of the device once (the
    MI355X this library is tuned on has 256; so does a host without a GPU, for the tests of the
    launch shapes).  The shape thresholds of ``skinny_plan`` are measured on that part."""
    if not torch.cuda.is_available():
        return 256
    idx = torch.cuda.current_device() if device is None else torch.device(device).index or 0
    if idx not in _COMPUTE_UNITS:
        _COMPUTE_UNITS[idx] = int(torch.cuda.get_device_properties(idx).multi_processor_count)
    return _COMPUTE_UNITS[idx]


def _row_blocks(group_rows: Optional[int]) -> int:
    """16-row blocks of one expert that a grouped launch multiplies at a time: enough for the
    largest group (its bound is the caller's), 1, 2 or 4; larger groups are walked in turns."""
    if not group_rows or group_rows <= 16:
        return 1
    return 2 if group_rows <= 32 else 4


def gemm_skinny(x: torch.Tensor, w, out_dtype: torch.dtype, a_rows: Optional[torch.Tensor] = None,
                offsets: Optional[torch.Tensor] = None, n_rows: Optional[int] = None, R: Optional[int] = None,
                NW: Optional[int] = None, group_rows: Optional[int] = None) -> torch.Tensor:
    """x [M, K] @ w[N, K]^T for M <= 64, or per expert with w [E, N, K] over an expert-sorted row
    list (``group_rows``: a bound on the rows of one expert, if known), on the matrix cores;
    w a tensor (row-major) or a PackedWeight."""
    w, packed = _unwrap(w)
    _dev(x, w, a_rows, offsets)
    _i32(a_rows, "a_rows")
    _i32(offsets, "offsets")
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_skinny: bfloat16 operands only")
    grouped = offsets is not None
    if grouped:
        _need(w.dim() == 3 and 2 <= offsets.shape[0] <= w.shape[0] + 1,
              "gemm_skinny: grouped needs w [E, N, K] and offsets of at most E + 1 entries")
        E, N, K = offsets.shape[0] - 1, w.shape[1], w.shape[2]
        M = int(n_rows)
        if a_rows is not None:
            _need(a_rows.shape == (M,), "gemm_skinny: a_rows must be [n_rows]")
        else:
            _need(x.shape[0] == M, "gemm_skinny: x must have n_rows rows when not gathered")
    else:
        _need(w.dim() == 2 and a_rows is None, "gemm_skinny: plain needs w [N, K]")
        E, (N, K) = 0, w.shape
        M = x.shape[0]
    _need(x.dim() == 2 and x.shape[1] == K, f"gemm_skinny: x {tuple(x.shape)} vs w {tuple(w.shape)}")
    _need(M > 0 and (grouped or M <= SKINNY_MAX_ROWS) and K % 128 == 0 and N % 4 == 0,
          f"gemm_skinny: shape M={M} N={N} K={K} is not taken (M <= 64 unless grouped, K % 128 == 0, N % 4 == 0)")
    pr, pw = skinny_plan(N, K, _row_blocks(group_rows) if grouped else (M + 15) // 16, max(E, 1))
    out = torch.empty(M, N, dtype=out_dtype, device=x.device)
    _run("sharpi_gemm_skinny", _ptr(x), _ptr(w), _ptr(out), _code(out_dtype), M, N, K, _ptr(a_rows), _ptr(offsets), E,
         R or pr, NW or pw, 1 if packed else 0, _row_blocks(group_rows) if grouped else 0, _stream())
    return out


def gemm_skinny_swiglu(x: torch.Tensor, w, offsets: torch.Tensor, a_rows: Optional[torch.Tensor],
                       n_rows: int, scale: Optional[torch.Tensor], R: Optional[int] = None,
                       NW: Optional[int] = None, group_rows: Optional[int] = None, act=ACT_SILU) -> torch.Tensor:
    """Per expert, silu(s g) * (s u) with (g | u) = x @ w[e]^T rounded to bfloat16, w [E, 2I, K]
    holding gate rows then up rows: the product and the activation in one kernel, for at most
    64 rows.  Returns [n_rows, I] bfloat16."""
    w, packed = _unwrap(w)
    _dev(x, w, a_rows, offsets, scale)
    _i32(a_rows, "a_rows")
    _i32(offsets, "offsets")
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_skinny_swiglu: bfloat16 operands only")
    _need(w.dim() == 3 and 2 <= offsets.shape[0] <= w.shape[0] + 1,
          "gemm_skinny_swiglu: w [E, 2I, K] and offsets of at most E + 1 entries")
    E, N, K = offsets.shape[0] - 1, w.shape[1], w.shape[2]
    M = int(n_rows)
    if a_rows is not None:
        _need(a_rows.shape == (M,), "gemm_skinny_swiglu: a_rows must be [n_rows]")
    else:
        _need(x.shape[0] == M, "gemm_skinny_swiglu: x must have n_rows rows when not gathered")
    _need(x.dim() == 2 and x.shape[1] == K, f"gemm_skinny_swiglu: x {tuple(x.shape)} vs w {tuple(w.shape)}")
    _need(M > 0 and K % 128 == 0 and N % 8 == 0,
          f"gemm_skinny_swiglu: shape M={M} N={N} K={K} is not taken (K % 128 == 0, N % 8 == 0)")
    _need(not packed or N % 32 == 0, "gemm_skinny_swiglu: packed weights need gate and up rows in whole 16-row tiles")
    if scale is not None:
        _need(scale.dtype == torch.float32 and scale.shape == (M,), "gemm_skinny_swiglu: scale must be float32 [n_rows]")
    pr, pw = skinny_plan(N, K, _row_blocks(group_rows), E, act=True)
    out = torch.empty(M, N // 2, dtype=torch.bfloat16, device=x.device)
    _run("sharpi_gemm_skinny_swiglu", _ptr(x), _ptr(w), _ptr(out), M, N, K, _ptr(a_rows), _ptr(offsets), E,
         _ptr(scale), R or pr, NW or pw, 1 if packed else 0, _row_blocks(group_rows), *_act_pair(act), _stream())
    return out


ROUTER_MAX_EXPERTS = _lib.ROUTER_MAX_EXPERTS   # experts the routing kernels hold scores for (csrc/router.hip kMaxExperts)
PICKED_MAX_PAIRS = _lib.PICKED_MAX_PAIRS   # (token, pick) pairs of the picked form: one ballot of a wave (csrc/gemm_skinny_kernel.h kMaxPicked)

_COUNTING: dict = {}    # per device: 0, 1, 2, ... (the places of pairs that are stored in their own order)


def counting(n: int, dev: torch.device) -> torch.Tensor:
    """int32 [n] = 0 .. n-1 on the device, from one tensor per device that is made once (outside
    any graph capture)."""
    c = _COUNTING.get(dev)
    if c is None or c.numel() < n:
        _need(not torch.cuda.is_current_stream_capturing(), "counting: the first call on a device must not be captured")
        c = _COUNTING[dev] = torch.arange(max(n, 4096), dtype=torch.int32, device=dev)
    return c[:n]


def picked_ok(n_tokens: int, k: int, N: int, K: int, act: bool, packed: bool) -> bool:
    return (0 < n_tokens * k <= PICKED_MAX_PAIRS and K % 128 == 0
            and N % ((32 if packed else 8) if act else (16 if packed else 4)) == 0)


def gemm_skinny_picked(x: torch.Tensor, w, ids: torch.Tensor, wts: Optional[torch.Tensor], shared: bool, gather: bool,
                       act, out_dtype: torch.dtype) -> torch.Tensor:
    """Per-expert products of a few decode tokens straight from the router's picks ids [T, k]:
    row i of the result is pair i = (token i // k, pick i % k), followed (shared) by one row per
    token through expert E of w [E + 1, N, K].  gather: x [T, K] is read by token, otherwise x is in
    the result's row order.  act (True: SiLU; or an activation's code; False: none): w holds gate
    rows then up rows and the result is act(s g) * (s u) [rows, N/2] with s the pair's weight (wts;
    1 for the shared rows)."""
    act, act_limit = _act_pair(ACT_SILU if act is True else act)
    w, packed = _unwrap(w)
    _dev(x, w, ids, wts)
    _i32(ids, "ids")
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_skinny_picked: bfloat16 operands only")
    _need(ids.dim() == 2 and ids.is_contiguous(), "gemm_skinny_picked: ids [T, k]")
    T, k = ids.shape
    E = w.shape[0] - (1 if shared else 0)
    _need(w.dim() == 3 and E >= 1, "gemm_skinny_picked: w [E (+ 1), N, K]")
    N, K = w.shape[1], w.shape[2]
    _need(picked_ok(T, k, N, K, act, packed), f"gemm_skinny_picked: T={T} k={k} N={N} K={K} is not taken")
    rows = T * k + (T if shared else 0)
    _need(x.dim() == 2 and x.shape[1] == K and x.shape[0] == (T if gather else rows),
          f"gemm_skinny_picked: x {tuple(x.shape)} has the wrong shape")
    if wts is not None:
        _need(act and wts.dtype == torch.float32 and wts.shape == ids.shape and wts.is_contiguous(),
              "gemm_skinny_picked: weights are float32 [T, k] and belong to the activation form")
    if act:
        _need(out_dtype == torch.bfloat16, "gemm_skinny_picked: the activation form stores bfloat16")
    # (row blocks: the kernel's own rule; groups: what it launches)
    pr, pw = skinny_plan(N, K, 1 if T * k <= 16 else 2 if T * k <= 32 else 4, min(E, T * k) + (1 if shared else 0), bool(act))
    out = torch.empty(rows, N // 2 if act else N, dtype=out_dtype, device=x.device)
    _run("sharpi_gemm_skinny_picked", _ptr(x), _ptr(w), _ptr(out), _code(out_dtype), N, K, _ptr(ids), _ptr(wts), T * k, k, E,
         1 if shared else 0, 1 if gather else 0, act, act_limit, pr, pw, 1 if packed else 0, _stream())
    return out


def linear(x: torch.Tensor, w, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """y = x W^T.  float32 weights: the float FMA kernel (true 32-bit, whatever x was stored
    as).  bfloat16 weights stored tile by tile (a PackedWeight): the weight-streaming kernel for a
    few rows; beyond, the library's matrix product with float accumulation over the row-major
    copy, as the reference calls a library there (reference:
    src/SharpInference.Cuda/CuBlasInterop.cs:55-68; measured, the library is at the matrix cores'
    peak for plain shapes), or, where only the packed copy is kept, this library's own kernels
    (the few-rows kernel up to 64 rows, the grouped kernel with the matrix as its one group
    beyond)."""
    out_dtype = out_dtype or x.dtype
    if isinstance(w, PackedWeight):
        xb = x if x.dtype == torch.bfloat16 else cast(x, torch.bfloat16)
        _need(xb.dim() == 2 and xb.shape[1] == w.shape[1], f"linear: x {tuple(x.shape)} vs w {tuple(w.shape)}")
        M, (N, K) = xb.shape[0], w.shape
        if skinny_ok(M, N, K):
            return gemm_skinny(xb, w, out_dtype)
        if w.rows is None:
            # only the packed copy is kept (the engine was asked to save memory): this library's own kernels
            if M <= SKINNY_MAX_ROWS:
                return gemm_skinny(xb, w, out_dtype)
            if dense_grouped_ok(M, N, K):
                return linear_many_rows(xb, w, out_dtype)
        w = unpack_weight(w)
    if w.dtype == torch.float32:
        xf = x if x.dtype == torch.float32 else cast(x, torch.float32)
        y = gemm_tiled(xf, w, torch.float32)
        return y if out_dtype == torch.float32 else cast(y, out_dtype)
    _dev(x, w)
    xb = x if x.dtype == torch.bfloat16 else cast(x, torch.bfloat16)
    _need(xb.shape[1] == w.shape[1], f"linear: x {tuple(x.shape)} vs w {tuple(w.shape)}")
    if skinny_ok(xb.shape[0], w.shape[0], w.shape[1]):
        return gemm_skinny(xb, w, out_dtype)
    if out_dtype == torch.bfloat16:
        return torch.mm(xb, w.t())
    return torch.mm(xb, w.t(), out_dtype=torch.float32)


def grouped_gemm(x: torch.Tensor, w: torch.Tensor, offsets: torch.Tensor, a_rows: Optional[torch.Tensor],
                 n_rows: int) -> torch.Tensor:
    """Rows [offsets[e], offsets[e+1]) of the expert-sorted list times w[e]^T.
    x rows are read through a_rows when given; w is [E, N, K]; returns [n_rows, N]."""
    _dev(x, w, offsets, a_rows)
    _i32(offsets, "offsets")
    _i32(a_rows, "a_rows")
    _need(w.dim() == 3 and x.dim() == 2 and x.shape[1] == w.shape[2] and x.dtype == w.dtype,
          f"grouped_gemm: x {tuple(x.shape)} vs w {tuple(w.shape)}")
    N, K = w.shape[1], w.shape[2]
    E = offsets.shape[0] - 1          # the weight may hold more experts than the routing has groups
    _need(1 <= E <= w.shape[0], "grouped_gemm: offsets must have at most E + 1 entries")
    if a_rows is not None:
        _need(a_rows.shape == (n_rows,), "grouped_gemm: a_rows must be [n_rows]")
    else:
        _need(x.shape[0] == n_rows, "grouped_gemm: x must have n_rows rows when not gathered")
    out = torch.empty(n_rows, N, dtype=x.dtype, device=x.device)
    _run("sharpi_gemm_tiled", _ptr(x), _ptr(w), _ptr(out), _code(x.dtype), _code(x.dtype), n_rows, N, K, _ptr(a_rows),
         _ptr(offsets), E, _stream())
    return out


# ---------------------------------------------------------------------------
GATE_SIGMOID, GATE_SOFTMAX, GATE_SOFTMAX_PICKED = 0, 1, 2


def router_topk(x: torch.Tensor, wr: torch.Tensor, k: int, gate: int = GATE_SIGMOID, renorm: bool = False,
                want_gates: bool = False, correction: Optional[torch.Tensor] = None, n_groups: int = 1,
                keep_groups: int = 1, bias: Optional[torch.Tensor] = None):
    """Router logits in float (plus ``bias``, float32 [E], where given), gate, k picks (lowest index
    wins a tie).  Gates: sigmoid, softmax over all experts, or GATE_SOFTMAX_PICKED: the largest logits are
    picked and the weights are the softmax over the picked logits alone (the gate values handed
    out are then the logits).
    Returns ids int32 [T, k], weights float32 [T, k] (and the gate values [T, E] if asked).
    ``correction`` (float32 [E]) is added to the gate values for the choice only: the weights stay
    the gate values.  With ``n_groups`` > ``keep_groups`` the experts form n_groups equal groups of
    neighbours and only those of the keep_groups best groups can be picked (a group's rank: the sum
    of its two largest choice scores)."""
    _dev(x, wr, correction, bias)
    _need(x.dim() == 2 and wr.dim() == 2 and x.shape[1] == wr.shape[1], "router: x [T, H], wr [E, H]")
    T, H = x.shape
    E = wr.shape[0]
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (E,), "router: bias must be float32 [E]")
    if correction is not None:
        _need(correction.dtype == torch.float32 and correction.shape == (E,), "router: correction must be float32 [E]")
    _need(1 <= keep_groups <= n_groups and E % n_groups == 0 and k <= keep_groups * (E // n_groups),
          f"router: {n_groups} groups (keep {keep_groups}) do not fit {E} experts and {k} picks")
    ids = torch.empty(T, k, dtype=torch.int32, device=x.device)
    wts = torch.empty(T, k, dtype=torch.float32, device=x.device)
    gates = torch.empty(T, E, dtype=torch.float32, device=x.device) if want_gates else None
    _run("sharpi_router_topk", _ptr(x), _code(x.dtype), _ptr(wr), _code(wr.dtype), _ptr(ids), _ptr(wts), _ptr(gates),
         T, H, E, k, gate, 1 if renorm else 0, _ptr(correction), int(n_groups), int(keep_groups), _ptr(bias), _stream())
    return (ids, wts, gates) if want_gates else (ids, wts)


FUSED_NORM_ROUTER_MAX_HIDDEN = _lib.FUSED_NORM_ROUTER_MAX_HIDDEN   # csrc/router.hip kFusedMaxHidden


def norm_router_ok(h: torch.Tensor, delta, out_dtype: torch.dtype) -> bool:
    """Can add_rmsnorm_router take this step?  (a plain bfloat16 delta or none, a width the
    kernel's LDS row holds)"""
    return (out_dtype == torch.bfloat16 and h.shape[1] % 8 == 0 and h.shape[1] <= FUSED_NORM_ROUTER_MAX_HIDDEN
            and (delta is None or (isinstance(delta, torch.Tensor) and delta.dtype == torch.bfloat16
                                   and delta.is_contiguous() and tuple(delta.shape) == tuple(h.shape))))


def add_rmsnorm_router(h: torch.Tensor, delta: Optional[torch.Tensor], weight: Optional[torch.Tensor], eps: float,
                       wr: torch.Tensor, k: int, gate: int = GATE_SIGMOID, renorm: bool = False):
    """add_rmsnorm (the sum goes back into h) and router_topk on its output in one launch, for a
    few tokens: returns (normalised rows bfloat16 [T, H], ids [T, k], weights [T, k]), the bits
    of the two kernels in a row."""
    _dev(h, delta, weight, wr)
    _need(h.dim() == 2 and h.dtype == torch.float32, "add_rmsnorm_router: h must be float32 [T, H]")
    T, H = h.shape
    _need(norm_router_ok(h, delta, torch.bfloat16), "add_rmsnorm_router: bfloat16 rows of a width the kernel holds only")
    if delta is not None:
        _need(tuple(delta.shape) == (T, H) and delta.is_contiguous(), "add_rmsnorm_router: delta must be [T, H]")
    if weight is not None:
        _need(weight.shape == (H,), f"add_rmsnorm_router: weight {tuple(weight.shape)} vs width {H}")
    _need(wr.dim() == 2 and wr.shape[1] == H, "add_rmsnorm_router: wr [E, H]")
    E = wr.shape[0]
    out = torch.empty(T, H, dtype=torch.bfloat16, device=h.device)
    ids = torch.empty(T, k, dtype=torch.int32, device=h.device)
    wts = torch.empty(T, k, dtype=torch.float32, device=h.device)
    _run("sharpi_add_rmsnorm_router", _ptr(h), _ptr(delta), _ptr(weight), _code(weight.dtype) if weight is not None else 0,
         _ptr(out), T, H, float(eps), _ptr(wr), _code(wr.dtype), _ptr(ids), _ptr(wts), E, k, gate, 1 if renorm else 0,
         _stream())
    return out, ids, wts




class Routing:
    """The expert-sorted view of a step's (token, pick) pairs, all on the device."""

    __slots__ = ("n_tokens", "k", "n_experts", "n_groups", "offsets", "sorted_token", "sorted_w", "inv_pos", "plan")

    @property
    def n_rows(self) -> int:
        """Rows of the sorted list: one per (token, pick), plus one per token for a shared group."""
        return self.n_tokens * self.k + (self.n_tokens if self.n_groups > self.n_experts else 0)


_PLAN_INTS: dict = {}


def _new_routing(T: int, k: int, n_experts: int, shared_group: bool, dev) -> Routing:
    rt = Routing()
    rt.n_tokens, rt.k, rt.n_experts = T, k, n_experts
    rt.n_groups = n_experts + (1 if shared_group else 0)
    rows = T * k + (T if shared_group else 0)
    if rt.n_groups not in _PLAN_INTS:
        _PLAN_INTS[rt.n_groups] = _lib.grouped_plan_ints(rt.n_groups)
    n_plan = _PLAN_INTS[rt.n_groups]
    ints = torch.empty(rt.n_groups + 1 + rows + T * k + n_plan, dtype=torch.int32, device=dev)
    o = 0
    rt.offsets = ints[o:o + rt.n_groups + 1]; o += rt.n_groups + 1
    rt.sorted_token = ints[o:o + rows]; o += rows
    rt.inv_pos = ints[o:o + T * k]; o += T * k
    rt.plan = ints[o:o + n_plan]
    rt.sorted_w = torch.empty(rows, dtype=torch.float32, device=dev)
    return rt


def moe_permute(ids: torch.Tensor, wts: torch.Tensor, n_experts: int, shared_group: bool = False) -> Routing:
    """(token, pick) pairs sorted by expert: offsets [E+1], sorted_token, sorted_w, inv_pos, and
    the plan of the grouped product for many rows, which
    says how the experts' row tiles are dealt to the blocks (csrc/grouped_plan.h).  With
    shared_group one more group follows the experts: every token once with weight 1."""
    _dev(ids, wts)
    _i32(ids, "ids")
    _need(ids.shape == wts.shape and wts.dtype == torch.float32 and ids.dim() == 2, "moe_permute: ids/wts [T, k]")
    T, k = ids.shape
    rt = _new_routing(T, k, n_experts, shared_group, ids.device)
    _run("sharpi_moe_permute", _ptr(ids), _ptr(wts), _ptr(rt.offsets), _ptr(rt.sorted_token), _ptr(rt.sorted_w),
         _ptr(rt.inv_pos), _ptr(rt.plan), rt.plan.numel(), T, k, n_experts,
         1 if shared_group else 0, _stream())
    return rt


def route(x: torch.Tensor, wr: torch.Tensor, k: int, gate: int = GATE_SIGMOID, renorm: bool = False,
          shared_group: bool = False, correction: Optional[torch.Tensor] = None, n_groups: int = 1,
          keep_groups: int = 1, bias: Optional[torch.Tensor] = None):
    """router_topk then moe_permute: (ids, weights, Routing)."""
    ids, wts = router_topk(x, wr, k, gate, renorm, correction=correction, n_groups=n_groups, keep_groups=keep_groups,
                           bias=bias)
    return ids, wts, moe_permute(ids, wts, wr.shape[0], shared_group)


def gemm_grouped(x: torch.Tensor, w, rt: Routing, gather: bool, out_dtype: torch.dtype, max_blocks: int = 0) -> torch.Tensor:
    """Per-group products for many rows on the matrix cores (bfloat16): the experts, and the
    always-on group if the routing has one (group E of w).  gather: x rows are read through the
    routing's token list; otherwise x is already in expert-sorted order.  The product's blocks
    stay on their compute units until the work is done; ``max_blocks`` > 0 bounds their number
    (the units left over are for other work running beside the product).  Products that read
    one routing must not run at the same time (they share its plan's ticket counters)."""
    w, packed = _unwrap(w)
    _dev(x, w)
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_grouped: bfloat16 operands only")
    _need(w.dim() == 3 and w.shape[0] >= rt.n_groups and x.dim() == 2 and x.shape[1] == w.shape[2],
          f"gemm_grouped: x {tuple(x.shape)} vs w {tuple(w.shape)}")
    E, N, K = w.shape
    _need(K % 64 == 0 and N % 4 == 0, "gemm_grouped: K % 64 == 0 and N % 4 == 0 wanted")
    _need(x.shape[0] == (rt.n_tokens if gather else rt.n_rows), "gemm_grouped: x has the wrong number of rows")
    out = torch.empty(rt.n_rows, N, dtype=out_dtype, device=x.device)
    _run("sharpi_gemm_grouped", _ptr(x), x.shape[0], _ptr(w), _ptr(out), _code(out_dtype), rt.n_rows, N, K,
         _ptr(rt.sorted_token) if gather else None, _ptr(rt.offsets), _ptr(rt.plan), rt.n_groups,
         1 if packed else 0, int(max_blocks), _stream())
    return out


def gemm_grouped_swiglu(x: torch.Tensor, w, rt: Routing, scale: Optional[torch.Tensor], gather: bool = True,
                        act=ACT_SILU, max_blocks: int = 0) -> torch.Tensor:
    """Per group, act(s g) * (s u) with (g | u) = x @ w[e]^T rounded to bfloat16, for many rows: the
    grouped product with the activation (ACT_SILU, ACT_GELU_TANH) in its epilogue.  gather: x rows are read through the
    routing's token list (the order inside a group is whatever the routing kernel made it);
    otherwise x is already in the groups' order.  w [E (+ 1), 2I, K] holds gate rows then up
    rows.  Returns [n_rows, I] bfloat16."""
    w, packed = _unwrap(w)
    _dev(x, w, scale)
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_grouped_swiglu: bfloat16 operands only")
    _need(w.dim() == 3 and w.shape[0] >= rt.n_groups and x.dim() == 2 and x.shape[1] == w.shape[2],
          f"gemm_grouped_swiglu: x {tuple(x.shape)} vs w {tuple(w.shape)}")
    E, N, K = w.shape
    _need(K % 64 == 0 and N % 32 == 0, "gemm_grouped_swiglu: K % 64 == 0 and N % 32 == 0 wanted")
    _need(x.shape[0] == (rt.n_tokens if gather else rt.n_rows), "gemm_grouped_swiglu: x has the wrong number of rows")
    if scale is not None:
        _need(scale.dtype == torch.float32 and scale.shape == (rt.n_rows,), "gemm_grouped_swiglu: scale must be float32 [n_rows]")
    out = torch.empty(rt.n_rows, N // 2, dtype=torch.bfloat16, device=x.device)
    _run("sharpi_gemm_grouped_swiglu", _ptr(x), x.shape[0], _ptr(w), _ptr(out), rt.n_rows, N, K,
         _ptr(rt.sorted_token) if gather else None, _ptr(rt.offsets), _ptr(rt.plan), rt.n_groups, _ptr(scale), 1 if packed else 0,
         *_act_pair(act), int(max_blocks), _stream())
    return out


# ---------------------------------------------------------------------------
# plain products of many rows through the grouped kernel (one group: the whole matrix)
# ---------------------------------------------------------------------------
_DENSE_ROUTING: "collections.OrderedDict" = collections.OrderedDict()
_DENSE_ROUTING_KEPT = 64


def _dense_routing(T: int, dev: torch.device) -> Routing:
    """The routing of T rows that all belong to one group: offsets [0, T] and the plan of the
    grouped product for it, made by the routing kernel when a row count is first met and kept for
    the row counts used last (the least recently used one gives way).  Its token list is not used
    (the routing kernel promises no order inside a group): the products read x row by row
    (gather off)."""
    key = (T, dev)
    rt = _DENSE_ROUTING.get(key)
    if rt is None:
        _need(not torch.cuda.is_current_stream_capturing(), "a dense routing's first use must not be captured")
        while len(_DENSE_ROUTING) >= _DENSE_ROUTING_KEPT:
            _DENSE_ROUTING.popitem(last=False)
        ids = torch.zeros(T, 1, dtype=torch.int32, device=dev)
        rt = _DENSE_ROUTING[key] = moe_permute(ids, torch.ones(T, 1, dtype=torch.float32, device=dev), 1)
    else:
        _DENSE_ROUTING.move_to_end(key)
    return rt


def dense_grouped_ok(M: int, N: int, K: int) -> bool:
    return M > 0 and K % 128 == 0 and N % 16 == 0 and N * K <= 0x7fffffff


def linear_many_rows(x: torch.Tensor, w: PackedWeight, out_dtype: torch.dtype) -> torch.Tensor:
    """x [M, K] @ w^T for many rows against a matrix stored tile by tile, on the matrix cores: the
    grouped product with the whole matrix as its one group (row tiles of up to 128 rows whose
    blocks share the weight stream through an XCD's L2)."""
    rt = _dense_routing(x.shape[0], x.device)
    return gemm_grouped(x, PackedWeight(w.packed.unsqueeze(0), None), rt, False, out_dtype)


def swiglu_many_rows(x: torch.Tensor, w_gate_up: PackedWeight, act: int = ACT_SILU) -> torch.Tensor:
    """silu(g) * u with (g | u) = x @ w_gate_up^T rounded to bfloat16, for many rows, the activation
    in the product's epilogue: [M, I] bfloat16."""
    rt = _dense_routing(x.shape[0], x.device)
    return gemm_grouped_swiglu(x, PackedWeight(w_gate_up.packed.unsqueeze(0), None), rt, None, gather=False, act=act)


# ---------------------------------------------------------------------------
def argmax_rows(logits: torch.Tensor) -> torch.Tensor:
    _dev(logits)
    _need(logits.dim() == 2 and logits.dtype == torch.float32, "argmax: logits must be float32 [rows, vocab]")
    out = torch.empty(logits.shape[0], dtype=torch.int32, device=logits.device)
    _run("sharpi_argmax_rows", _ptr(logits), _ptr(out), logits.shape[0], logits.shape[1], _stream())
    return out


def sample_rows(logits: torch.Tensor, temperature: torch.Tensor, uniform: torch.Tensor,
                top_k: Optional[torch.Tensor] = None, top_p: Optional[torch.Tensor] = None,
                min_p: Optional[torch.Tensor] = None) -> torch.Tensor:
    _dev(logits, temperature, uniform, top_k, top_p, min_p)
    _need(logits.dim() == 2 and logits.dtype == torch.float32, "sample: logits must be float32 [rows, vocab]")
    R = logits.shape[0]
    for name, t, dt in (("temperature", temperature, torch.float32), ("uniform", uniform, torch.float32),
                        ("top_k", top_k, torch.int32), ("top_p", top_p, torch.float32), ("min_p", min_p, torch.float32)):
        if t is not None:
            _need(t.shape == (R,) and t.dtype == dt, f"sample: {name} must be {dt} [rows]")
    probs = torch.empty_like(logits)
    out = torch.empty(R, dtype=torch.int32, device=logits.device)
    _run("sharpi_sample_rows", _ptr(logits), _ptr(probs), _ptr(temperature), _ptr(uniform), _ptr(top_k), _ptr(top_p),
         _ptr(min_p), _ptr(out), R, logits.shape[1], _stream())
    return out


def edit_logits(logits: torch.Tensor, row_offsets: torch.Tensor, ids: torch.Tensor, counts: torch.Tensor,
                bias: torch.Tensor, rep: torch.Tensor, freq: torch.Tensor, pres: torch.Tensor) -> None:
    _dev(logits, row_offsets, ids, counts, bias, rep, freq, pres)
    _need(logits.dim() == 2 and logits.dtype == torch.float32, "edit_logits: logits must be float32 [rows, vocab]")
    R = logits.shape[0]
    _i32(row_offsets, "row_offsets"); _i32(ids, "ids"); _i32(counts, "counts")
    _need(row_offsets.shape == (R + 1,), "edit_logits: row_offsets must be [rows + 1]")
    n = ids.shape[0]
    _need(counts.shape == (n,) and bias.shape == (n,) and bias.dtype == torch.float32, "edit_logits: per-entry arrays")
    for t in (rep, freq, pres):
        _need(t.shape == (R,) and t.dtype == torch.float32, "edit_logits: per-row arrays must be float32 [rows]")
    _run("sharpi_edit_logits", _ptr(logits), _ptr(row_offsets), _ptr(ids), _ptr(counts), _ptr(bias), _ptr(rep),
         _ptr(freq), _ptr(pres), R, logits.shape[1], _stream())


# ---------------------------------------------------------------------------
# between the projections and attention, for layers that norm before they rotate
# ---------------------------------------------------------------------------
NORM_NONE, NORM_PER_HEAD, NORM_WHOLE = 0, 1, 2
QK_PREP_MAX_TAPS = 8          # csrc/qk_prep.hip kPrepMaxTaps
QK_PREP_MAX_ROW = 15 * 1024   # q + k + v channels of a token that the kernel holds in LDS as floats


def qk_prep(proj: torch.Tensor, q_off: int, k_off: int, v_off: Optional[int], nh: int, nkv: int, hd: int, vd: int,
            ctx, k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], slot_mapping: Optional[torch.Tensor],
            norm_mode: int = NORM_NONE, q_norm_w: Optional[torch.Tensor] = None, k_norm_w: Optional[torch.Tensor] = None,
            eps: float = 1e-6, inv_freq: Optional[torch.Tensor] = None, pair_layout: int = PAIRS_INTERLEAVED,
            magnitude: float = 1.0, conv_w: Optional[torch.Tensor] = None, tail: Optional[torch.Tensor] = None,
            update_tail: bool = True, bias: Optional[torch.Tensor] = None,
            temperature: Optional[Tuple[float, float]] = None, maps: int = 1) -> torch.Tensor:
    """From a step's projections proj [T, N] (q at columns q_off.., k at k_off.., v at v_off.., or
    v_off None: the values are the keys before norm and rotation): optional short causal
    convolution over time on every channel (conv_w float32 [channels, taps]; tail float32 [slots,
    taps - 1, channels] carries each request's last projected rows from step to step and is brought
    up to date unless update_tail is False), RMS norm of q and k with learned weights (per head, or
    over the whole projection), rotary positions (cos and sin times `magnitude`), keys and values
    into the cache at slot_mapping (None: nothing is stored).  Returns q [T, nh*hd].

    ``bias`` (float32, one value per channel of q, k and v; only without a convolution) is added to the
    row as it is read.  ``temperature`` = (floor_scale, attn_scale) multiplies q by
    1 + attn_scale * ln(floor((pos + 1) / floor_scale) + 1).  ``maps`` > 1: a head holds that many score
    maps side by side (hd is their width together; rotary_dim at most hd / maps, applied to each map's
    own leading elements), and q comes back expanded, [T, nh * maps * hd]: one row of the head's width
    per (head, map), the map's elements in their place and zeros elsewhere, so that attention over
    nh * maps query heads and keys of width hd computes every map's scores on its own."""
    _dev(proj, k_cache, v_cache, slot_mapping, q_norm_w, k_norm_w, inv_freq, conv_w, tail, bias)
    maps = int(maps)
    _need(maps >= 1 and hd % (2 * maps) == 0, "qk_prep: a head must split into its maps, each of even width")
    _i32(slot_mapping, "slot_mapping")
    T, N = proj.shape
    own_v = v_off is not None
    qn, kn, vn = nh * hd, nkv * hd, (nkv * vd if own_v else 0)
    _need(proj.dim() == 2 and 0 <= q_off and q_off + qn <= N and 0 <= k_off and k_off + kn <= N
          and (not own_v or (0 <= v_off and v_off + vn <= N)), "qk_prep: q, k and v columns must lie inside proj")
    _need(own_v or vd == hd, "qk_prep: values taken from the keys have the keys' width")
    _need(hd % 2 == 0 and qn + kn + vn <= QK_PREP_MAX_ROW, f"qk_prep: an even head size and at most {QK_PREP_MAX_ROW} channels a token")
    _need(ctx.positions.shape == (T,), "qk_prep: the step's positions must be [T]")
    if slot_mapping is not None:
        _need(slot_mapping.shape == (T,) and _cache_shapes_ok(k_cache, v_cache, nkv, hd, vd) and k_cache.dtype == proj.dtype
              and v_cache.dtype == proj.dtype, "qk_prep: slot_mapping [T]; caches K [pages, nkv, page_size, hd], V [pages, nkv, vd, page_size] of proj's dtype")
    _need(norm_mode in (NORM_NONE, NORM_PER_HEAD, NORM_WHOLE), "qk_prep: norm_mode 0, 1 or 2")
    if norm_mode != NORM_NONE:
        want_q, want_k = ((hd,), (hd,)) if norm_mode == NORM_PER_HEAD else ((qn,), (kn,))
        _need(q_norm_w is not None and k_norm_w is not None and q_norm_w.dtype == torch.float32 and k_norm_w.dtype == torch.float32
              and tuple(q_norm_w.shape) == want_q and tuple(k_norm_w.shape) == want_k,
              f"qk_prep: norm weights must be float32 {want_q} and {want_k}")
    rotary_dim = 0
    if inv_freq is not None:
        _need(inv_freq.dtype == torch.float32 and inv_freq.dim() == 1 and 1 <= inv_freq.shape[0] <= hd // 2,
              "qk_prep: inv_freq must be float32 [rotary_dim / 2], rotary_dim <= hd")
        rotary_dim = 2 * inv_freq.shape[0]
        _need(rotary_dim <= hd // maps, "qk_prep: the rotated width must fit one map of a head")
    if bias is not None:
        _need(conv_w is None and bias.dtype == torch.float32 and bias.shape == (qn + kn + vn,),
              "qk_prep: bias must be float32, one value per channel of q, k and v, and comes without a convolution")
    fs, asc = temperature if temperature is not None else (1.0, 0.0)
    _need(fs > 0, "qk_prep: the temperature's floor_scale must be positive")
    taps = 0
    if conv_w is not None:
        taps = conv_w.shape[1]
        _need(conv_w.dtype == torch.float32 and conv_w.shape == (qn + kn + vn, taps) and 2 <= taps <= QK_PREP_MAX_TAPS,
              f"qk_prep: conv_w must be float32 [q + k + v channels, 2..{QK_PREP_MAX_TAPS} taps]")
        _need(tail is not None and tail.dtype == torch.float32 and tail.dim() == 3 and tuple(tail.shape[1:]) == (taps - 1, qn + kn + vn),
              "qk_prep: tail must be float32 [slots, taps - 1, channels]")
        _need(ctx.state_slots.shape == (ctx.n_entries,) and ctx.cu_tokens.shape == (ctx.n_entries + 1,)
              and ctx.entry_of_token.shape == (T,), "qk_prep: the step's per-entry arrays do not fit")
    q_out = torch.empty(T, qn * maps, dtype=proj.dtype, device=proj.device)
    page_size = k_cache.shape[2] if k_cache is not None else 0
    _run("sharpi_qk_prep", _ptr(proj), _code(proj.dtype), N, int(q_off), int(k_off), int(v_off) if own_v else -1, T,
         ctx.n_entries, nh, nkv, hd, vd, _ptr(conv_w), taps, _ptr(tail), _ptr(ctx.state_slots), _ptr(ctx.entry_of_token),
         _ptr(ctx.cu_tokens), _ptr(ctx.positions), int(norm_mode), _ptr(q_norm_w), _ptr(k_norm_w), float(eps),
         _ptr(inv_freq), rotary_dim, 1 if pair_layout == PAIRS_HALF_SPLIT else 0, float(magnitude), _ptr(q_out),
         _ptr(k_cache), _ptr(v_cache), _ptr(slot_mapping), page_size, 1 if update_tail else 0, _ptr(bias),
         1 if temperature is not None else 0, float(fs), float(asc), maps, _stream())
    return q_out


# ---------------------------------------------------------------------------
# gated linear attention
# ---------------------------------------------------------------------------
GLA_MAX_KEY_DIM = 256      # key channels of a head that the walk holds (csrc/linear_attention.hip)
GLA_STATE_COLS = _lib.GLA_STATE_COLS   # value columns of the state that lie together in memory (checked against the library at load)


def _gla_rows(dk: int) -> int:
    """Rows of a state slice as the walk's lanes cover them: dk rounded up to 32, 64, 128 or 256."""
    return 32 if dk <= 32 else 64 if dk <= 64 else 128 if dk <= 128 else 256


def gla_state_shape(nh: int, dk: int, dv: int) -> tuple:
    """A request's recurrent state as the walk keeps it: [heads, ceil(dv / 8), DKP, 8], column slice by
    column slice, DKP = dk rounded up to 32 / 64 / 128 / 256; inside a slice row i = g * (DKP / 8) + r
    lies at place r * 8 + g (the order the walking wave's lanes hold it in)."""
    return (nh, (dv + GLA_STATE_COLS - 1) // GLA_STATE_COLS, _gla_rows(dk), GLA_STATE_COLS)


def gla_state_matrices(state: torch.Tensor, dk: int, dv: int) -> torch.Tensor:
    """The state as kept -> the matrices [.., heads, dk, dv] (a copy; for tests and tools)."""
    *lead, nh, ncb, dkp, c = state.shape
    rpl = dkp // 8
    m = state.reshape(*lead, nh, ncb, rpl, 8, c)                 # [.., h, slice, r, g, j]
    m = m.movedim(-2, -3)                                        # [.., h, slice, g, r, j]: row g * rpl + r
    m = m.reshape(*lead, nh, ncb, dkp, c).movedim(-3, -2)        # [.., h, row, slice, j]
    return m.reshape(*lead, nh, dkp, ncb * c)[..., :dk, :dv].contiguous()


def gla_decays(z: torch.Tensor, bias: torch.Tensor, tau: float) -> torch.Tensor:
    """Decay logits z float32 [T, N] turned IN PLACE into decays sigmoid(z + bias)^(1 / tau) (bias
    float32 [N]): log_sigmoid, the division by tau and the exponential in float."""
    _dev(z, bias)
    _need(z.dtype == torch.float32 and z.dim() == 2 and bias.dtype == torch.float32 and bias.shape == (z.shape[1],) and tau > 0,
          "gla_decays: z float32 [T, N], bias float32 [N], tau positive")
    _run("sharpi_gla_decays", _ptr(z), _ptr(bias), float(tau), z.shape[0], z.shape[1], _stream())
    return z


GLA_FUSED_DECAY_MAX_RANK = 256   # csrc/linear_attention.hip kDecayMaxRank


def gla_decays_from_middle(proj: torch.Tensor, a_off: int, rank: int, w: torch.Tensor, bias: torch.Tensor, tau: float) -> torch.Tensor:
    """Decays sigmoid(a1 w^T + bias)^(1 / tau), float32 [T, N], straight from the narrow middle a1 of
    their projection: columns a_off .. a_off + rank of proj [T, M]; w [N, rank] of proj's dtype, bias
    float32 [N].  One kernel: the product as ascending float chains, then log_sigmoid, the division
    by tau and the exponential in float."""
    _dev(proj, w, bias)
    T, M = proj.shape
    N = w.shape[0]
    _need(w.dtype == proj.dtype and w.shape == (N, rank) and 0 <= a_off and a_off + rank <= M and 1 <= rank <= GLA_FUSED_DECAY_MAX_RANK,
          f"gla_decays_from_middle: w [N, rank] of proj's dtype, rank 1..{GLA_FUSED_DECAY_MAX_RANK}, its columns inside proj")
    _need(bias.dtype == torch.float32 and bias.shape == (N,) and tau > 0, "gla_decays_from_middle: bias float32 [N], tau positive")
    alpha = torch.empty(T, N, dtype=torch.float32, device=proj.device)
    _run("sharpi_gla_decays_fused", _ptr(proj), _code(proj.dtype), M, int(a_off), int(rank), _ptr(w), _ptr(bias), float(tau),
         _ptr(alpha), T, N, _stream())
    return alpha


GLA_SEGMENT_TOKENS = 128       # tokens of a segment of the segmented walk


def gla_segments(lens, cu_tokens):
    """The work lists of the segmented walk for entries of `lens` tokens whose rows start at
    `cu_tokens`: (segs int32 [n, 4] = (entry, first row, tokens, 1 if the entry's last), ent_segs int32
    [entries, 2] = (first segment, segments)), as numpy arrays."""
    import numpy as np

    segs, ents = [], []
    for e, n in enumerate(lens):
        first = len(segs)
        for o in range(0, n, GLA_SEGMENT_TOKENS):
            m = min(GLA_SEGMENT_TOKENS, n - o)
            segs.append((e, int(cu_tokens[e]) + o, m, 1 if o + m == n else 0))
        ents.append((first, len(segs) - first))
    return np.asarray(segs, dtype=np.int32).reshape(-1, 4), np.asarray(ents, dtype=np.int32).reshape(-1, 2)


def gla_walk(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, alpha: torch.Tensor, q_scale: float,
             state: torch.Tensor, ctx, nh: int, dk: int, dv: int, segments=None) -> torch.Tensor:
    """The recurrence S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head, token by
    token along every entry of the step, from and into state [slots, *gla_state_shape(nh, dk, dv)]
    (float32) at the entries' state slots.  q, k (nh*dk columns each) and v (nh*dv) are columns of proj [T, N]; q is
    multiplied by q_scale; alpha float32 [T, nh*dk] are the decays.  Returns o float32 [T, nh*dv].
    ``segments`` = (segs, ent_segs) on the device (see :func:`gla_segments`): long entries are then walked
    segment by segment side by side (results equal to rounding)."""
    _dev(proj, alpha, state)
    T, N = proj.shape
    _need(1 <= dk <= GLA_MAX_KEY_DIM and dv >= 1 and nh >= 1, f"gla_walk: key channels 1..{GLA_MAX_KEY_DIM}")
    _need(min(q_off, k_off, v_off) >= 0 and max(q_off, k_off) + nh * dk <= N and v_off + nh * dv <= N,
          "gla_walk: q, k and v columns must lie inside proj")
    _need(alpha.dtype == torch.float32 and alpha.shape == (T, nh * dk), "gla_walk: alpha float32 [T, nh*dk] wanted")
    _need(state.dtype == torch.float32 and tuple(state.shape[1:]) == gla_state_shape(nh, dk, dv),
          "gla_walk: state must be float32 [slots, *gla_state_shape(nh, dk, dv)]")
    _need(ctx.state_slots.shape == (ctx.n_entries,) and ctx.cu_tokens.shape == (ctx.n_entries + 1,) and ctx.n_tokens == T,
          "gla_walk: the step's per-entry arrays do not fit")
    out = torch.empty(T, nh * dv, dtype=torch.float32, device=proj.device)
    if segments is not None:
        segs, ent_segs = segments
        _dev(segs, ent_segs)
        _i32(segs, "segs")
        _i32(ent_segs, "ent_segs")
        n_segs = segs.numel() // 4
        _need(segs.numel() == 4 * n_segs and ent_segs.numel() == 2 * ctx.n_entries and n_segs >= ctx.n_entries,
              "gla_walk: segs [n, 4] and ent_segs [entries, 2] wanted")
        seg_state = torch.empty((n_segs,) + gla_state_shape(nh, dk, dv), dtype=torch.float32, device=proj.device)
        seg_decay = torch.empty(n_segs, nh, _gla_rows(dk), dtype=torch.float32, device=proj.device)
        _run("sharpi_gla_walk_segmented", _ptr(proj), _code(proj.dtype), N, int(q_off), int(k_off), int(v_off), _ptr(alpha),
             float(q_scale), _ptr(state), _ptr(ctx.state_slots), _ptr(ctx.cu_tokens), _ptr(out), ctx.n_entries, nh, dk, dv,
             _ptr(segs), _ptr(ent_segs), n_segs, _ptr(seg_state), _ptr(seg_decay), _stream())
        return out
    _run("sharpi_gla_walk", _ptr(proj), _code(proj.dtype), N, int(q_off), int(k_off), int(v_off), _ptr(alpha),
         float(q_scale), _ptr(state), _ptr(ctx.state_slots), _ptr(ctx.cu_tokens), _ptr(out), ctx.n_entries,
         nh, dk, dv, int(getattr(ctx, "max_entry_len", 0) or T), _stream())
    return out


def head_norm_gate(o: torch.Tensor, weight: torch.Tensor, eps: float, nh: int, dv: int, out_dtype: torch.dtype,
                   gate_proj: Optional[torch.Tensor] = None, gate_off: int = 0) -> torch.Tensor:
    """o float32 [T, nh*dv] -> per (token, head) unit RMS over dv, times weight [dv] (shared by the
    heads), times silu of the gate (columns gate_off.. of gate_proj [T, N], of out_dtype; None: no gate)."""
    _dev(o, weight, gate_proj)
    T = o.shape[0]
    _need(o.dtype == torch.float32 and o.shape == (T, nh * dv) and weight.dtype == torch.float32 and weight.shape == (dv,),
          "head_norm_gate: o float32 [T, nh*dv], weight float32 [dv]")
    stride = 0
    if gate_proj is not None:
        _need(gate_proj.dtype == out_dtype and gate_proj.dim() == 2 and gate_proj.shape[0] == T
              and 0 <= gate_off and gate_off + nh * dv <= gate_proj.shape[1], "head_norm_gate: the gate's columns must lie inside gate_proj")
        stride = gate_proj.shape[1]
    out = torch.empty(T, nh * dv, dtype=out_dtype, device=o.device)
    _run("sharpi_head_norm_gate", _ptr(o), _ptr(weight), float(eps), _ptr(gate_proj), _code(out_dtype), stride, int(gate_off),
         _ptr(out), T, nh, dv, _stream())
    return out


class BranchMean:
    """Stands for the join of side-by-side branches, (1 / n) * sum_b unit_rms(xs[b]) * weights[b], still to
    be formed: float32 [T, N].  The norm kernel behind the branches forms it while it reads them
    (:func:`post_pre_norm`); ``tensor()`` forms it on its own for whoever needs a tensor."""

    def __init__(self, xs, weights, eps: float):
        self.xs, self.weights, self.eps = list(xs), list(weights), float(eps)
        self.shape, self.dtype = tuple(xs[0].shape), torch.float32

    def tensor(self) -> torch.Tensor:
        return norm_mean(self.xs, self.weights, self.eps)


POST_PRE_NORM_MAX_WIDTH = 15 * 1024     # floats of a row that the kernel keeps in LDS


def post_pre_norm(h: torch.Tensor, delta, w_post: torch.Tensor, eps: float, w_next: Optional[torch.Tensor] = None,
                  out_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """h += unit_rms(delta) * w_post in place in float, and, with w_next, returns unit_rms(new h) *
    w_next in out_dtype: the norm behind one branch and the norm before the next in one launch.
    delta: a tensor [T, N] or a BranchMean (formed by the kernel, with the eps of its own it was
    made with, which must equal eps).  Weights float32 [N]."""
    import ctypes

    lazy = delta if isinstance(delta, BranchMean) else None
    xs = lazy.xs if lazy is not None else [delta]
    ws = lazy.weights if lazy is not None else [None]
    _dev(h, w_post, w_next, *xs, *[w for w in ws if w is not None])
    _need(h.dim() == 2 and h.dtype == torch.float32, "post_pre_norm: h must be float32 [T, N]")
    T, N = h.shape
    _need(N <= POST_PRE_NORM_MAX_WIDTH and 1 <= len(xs) <= NORM_MEAN_MAX_BRANCHES, "post_pre_norm: row too wide or too many branches")
    _need(lazy is None or lazy.eps == float(eps), "post_pre_norm: the join was made with another eps")
    for x, w in zip(xs, ws):
        _need(tuple(x.shape) == (T, N) and x.dtype == xs[0].dtype and (w is None or (w.dtype == torch.float32 and w.shape == (N,))),
              "post_pre_norm: branches [T, N] of one dtype, weights float32 [N]")
    _need(w_post.dtype == torch.float32 and w_post.shape == (N,), "post_pre_norm: w_post must be float32 [N]")
    out = None
    if w_next is not None:
        _need(w_next.dtype == torch.float32 and w_next.shape == (N,) and out_dtype is not None, "post_pre_norm: w_next float32 [N] and an out_dtype")
        out = torch.empty(T, N, dtype=out_dtype, device=h.device)
    n = len(xs)
    xp = (ctypes.c_void_p * n)(*[x.data_ptr() for x in xs])
    wp = (ctypes.c_void_p * n)(*[(w.data_ptr() if w is not None else None) for w in ws])
    _run("sharpi_post_pre_norm", _ptr(h), ctypes.cast(xp, ctypes.c_void_p), ctypes.cast(wp, ctypes.c_void_p), n, _code(xs[0].dtype),
         _ptr(w_post), _ptr(w_next), _ptr(out), _code(out_dtype) if out is not None else 0, T, N, float(eps), _stream())
    return out


UNGATED_ACTIVATIONS = {"relu2": 1, "gelu_tanh": 2, "silu": 3}


def activation(x: torch.Tensor, name: str) -> torch.Tensor:
    """f(x) element by element, f one of UNGATED_ACTIVATIONS (relu2: the square of relu)."""
    _dev(x)
    _need(name in UNGATED_ACTIVATIONS, f"activation {name!r} is not known ({', '.join(sorted(UNGATED_ACTIVATIONS))})")
    out = torch.empty_like(x)
    _run("sharpi_activation", _ptr(x), _ptr(out), _code(x.dtype), x.numel(), UNGATED_ACTIVATIONS[name], _stream())
    return out


NORM_MEAN_MAX_BRANCHES = 4


def norm_mean(xs, weights, eps: float) -> torch.Tensor:
    """The mean over branches b of unit_rms(xs[b]) * weights[b], row by row: xs tensors [T, N] of one
    dtype, weights float32 [N].  Returns float32 [T, N]."""
    import ctypes

    n = len(xs)
    _need(1 <= n <= NORM_MEAN_MAX_BRANCHES and len(weights) == n, f"norm_mean: 1 to {NORM_MEAN_MAX_BRANCHES} branches, a weight vector each")
    _dev(*xs, *weights)
    T, N = xs[0].shape
    for x, w in zip(xs, weights):
        _need(x.shape == (T, N) and x.dtype == xs[0].dtype and w.dtype == torch.float32 and w.shape == (N,),
              "norm_mean: branches [T, N] of one dtype, weights float32 [N]")
    out = torch.empty(T, N, dtype=torch.float32, device=xs[0].device)
    xp = (ctypes.c_void_p * n)(*[x.data_ptr() for x in xs])
    wp = (ctypes.c_void_p * n)(*[w.data_ptr() for w in weights])
    _run("sharpi_norm_mean", ctypes.cast(xp, ctypes.c_void_p), ctypes.cast(wp, ctypes.c_void_p), n, _code(xs[0].dtype),
         _ptr(out), T, N, float(eps), _stream())
    return out


# ---------------------------------------------------------------------------
# dispatchers used by the parts
# ---------------------------------------------------------------------------
def attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, group, ctx, window_kind: int,
              window: int, scale: float, nh: int, nkv: int, hd: int, vd: Optional[int] = None, softcap: float = 0.0,
              sink=False) -> torch.Tensor:
    """Attention of the step's tokens over their requests' pages (`group`: the cache group's
    block tables, `ctx`: the step).  Values of another width than keys (vd) go through the float kernel.
    softcap > 0 caps the scores (softcap * tanh(score / softcap)); sink adds a key of score 0 without a
    value to the softmax's denominator (True), or one of a learned score per head (a float32 tensor [nh])."""
    same = vd is None or vd == hd
    if same and decode_attention_ok(q.dtype, hd) and (prefill_attention_ok(q.dtype, hd) or not ctx.n_prefill_tiles):
        # entries of one token: split-K decode kernel; longer entries: flash kernel, a tile of tokens a block
        out = torch.empty_like(q)
        if ctx.n_prefill_tiles:
            attention_prefill(q, k_cache, v_cache, group.block_table, ctx.positions, ctx.prefill_tiles, window_kind,
                              window, scale, nh, nkv, hd, out=out, tile_tokens=ctx.prefill_tile_tokens, softcap=softcap,
                              sink=sink)
        if ctx.n_decode:
            attention_decode(q, k_cache, v_cache, group.block_table, ctx.entry_of_token, ctx.positions,
                             ctx.decode_tokens, group.max_context, window_kind, window, scale, nh, nkv, hd, out=out,
                             softcap=softcap, sink=sink)
        return out
    return attention_generic(q, k_cache, v_cache, group.block_table, ctx.entry_of_token, ctx.positions, window_kind,
                             window, scale, nh, nkv, hd, vd, softcap=softcap, sink=sink)


def grouped_swiglu(x: torch.Tensor, w_gate_up, rt: Routing, out_dtype: torch.dtype, scaled: bool = True,
                   act=ACT_SILU, max_blocks: int = 0) -> torch.Tensor:
    """The experts' gate|up products of the routed tokens and their activation,
    act(s g) * (s u) with s the pick's weight (``scaled``; otherwise s = 1): [n_rows, I] in
    expert-sorted order.  On the matrix cores the activation is the product's epilogue (the
    few-rows kernel or the many-rows one); otherwise the product and the activation are two kernels."""
    N, K = w_gate_up.shape[1], w_gate_up.shape[2]
    scale = rt.sorted_w if scaled else None
    if x.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16 and out_dtype == torch.bfloat16 and K % 128 == 0:
        if rt.n_tokens <= SKINNY_MAX_ROWS and N % (32 if isinstance(w_gate_up, PackedWeight) else 8) == 0:
            return gemm_skinny_swiglu(x, w_gate_up, rt.offsets, rt.sorted_token, rt.n_rows, scale,
                                      group_rows=rt.n_tokens, act=act)
        if rt.n_tokens > SKINNY_MAX_ROWS and N % 32 == 0:
            return gemm_grouped_swiglu(x, w_gate_up, rt, scale, act=act, max_blocks=max_blocks)
    return gated_act(grouped_linear(x, w_gate_up, rt, True, out_dtype), scale, act)


def grouped_linear(x: torch.Tensor, w, rt: Routing, gather: bool, out_dtype: torch.dtype, max_blocks: int = 0) -> torch.Tensor:
    """Per-expert products over the routing's expert-sorted row list: w [E, N, K] (a tensor or a
    PackedWeight); x rows are read through the token list (gather) or are already in sorted order.
    Returns [n_rows, N]."""
    if x.dtype != w.dtype:
        x = cast(x, w.dtype)
    N, K = w.shape[1], w.shape[2]
    a_rows = rt.sorted_token if gather else None
    if w.dtype == torch.bfloat16 and K % 128 == 0 and N % 4 == 0:
        if rt.n_tokens <= SKINNY_MAX_ROWS:   # no expert has more rows than there are tokens
            return gemm_skinny(x, w, out_dtype, a_rows=a_rows, offsets=rt.offsets, n_rows=rt.n_rows,
                               group_rows=rt.n_tokens)
        return gemm_grouped(x, w, rt, gather, out_dtype, max_blocks=max_blocks)
    y = grouped_gemm(x, w, rt.offsets, a_rows, rt.n_rows)
    return y if y.dtype == out_dtype else cast(y, out_dtype)


# ---------------------------------------------------------------------------
# what the GPU gives at best (measured beside the published peaks)
# ---------------------------------------------------------------------------
def measured_peaks(device="cuda:0", read_bytes: int = 4 << 30, repeats: int = 5) -> dict:
    """{"hbm_gbs": GB/s of a pure read of `read_bytes`, "bf16_tflops": TFLOP/s of a resident loop of
    matrix-core products}: the best of `repeats` runs of two measuring kernels of this library."""
    dev = torch.device(device)
    buf = torch.empty(read_bytes, dtype=torch.uint8, device=dev)
    buf.fill_(1)
    sink = torch.zeros(4, dtype=torch.float32, device=dev)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best_read = best_mfma = float("inf")
    blocks, iters = 256 * 8, 4096
    import ctypes

    done = ctypes.c_longlong(0)
    for _ in range(repeats + 1):
        a.record()
        _run("sharpi_peak_read", _ptr(buf), read_bytes, _ptr(sink), ctypes.addressof(done), _stream())
        b.record()
        b.synchronize()
        best_read = min(best_read, a.elapsed_time(b))
        a.record()
        _run("sharpi_peak_mfma", _ptr(sink), blocks, iters, _stream())
        b.record()
        b.synchronize()
        best_mfma = min(best_mfma, a.elapsed_time(b))
    flops = blocks * 4 * iters * 8 * (2.0 * 16 * 16 * 32)
    return {"hbm_gbs": done.value / best_read / 1e6, "bf16_tflops": flops / best_mfma / 1e9}


# ---------------------------------------------------------------------------
# recurrent states with a scalar decay per (token, head); gated branches; a second input from the token
# ---------------------------------------------------------------------------
WALK_EXP_GATES, WALK_STATE_SPACE, WALK_FIXED_DECAY = 0, 1, 2      # csrc/state_walk.hip
WALK_MAX_KEY_DIM = 256
WALK_STATE_COLS = _lib.WALK_STATE_COLS
SHORT_CONV_MAX_TAPS = 8                       # csrc/state_walk.hip kConvMaxTaps
GATE_NONE, GATE_SILU, GATE_SIGMOID_ACT = 0, 1, 2


def _walk_rows(dk: int) -> int:
    return 32 if dk <= 32 else 64 if dk <= 64 else 128 if dk <= 128 else 256


def walk_state_shape(nh: int, dk: int, dv: int, mode: int) -> tuple:
    """A request's recurrent state as the walk keeps it: [heads, ceil(dv / 8), slice].  A slice holds 8
    value columns: DKP x 8 floats of the matrix (DKP = dk rounded up to 32 / 64 / 128 / 256; row
    g * (DKP / 8) + r of column j at r * 64 + 8 g + j) and, with exponential gates, DKP floats of the
    normaliser vector (four rows of a row group together, the groups side by side) and 8 floats that
    begin with the running maximum."""
    dkp = _walk_rows(dk)
    return (nh, (dv + WALK_STATE_COLS - 1) // WALK_STATE_COLS, dkp * 8 + (dkp + 8 if mode == WALK_EXP_GATES else 0))


def walk_state_matrices(state: torch.Tensor, dk: int, dv: int, mode: int):
    """The state as kept -> (S [.., heads, dk, dv], n [.., heads, dk] or None, m [.., heads] or None): copies, for
    tests and tools (the normaliser and the maximum are read from every head's first slice)."""
    *lead, nh, ncb, _ = state.shape
    dkp = _walk_rows(dk)
    rpl = dkp // 8
    S = state[..., : dkp * 8].reshape(*lead, nh, ncb, rpl, 8, 8)          # [.., h, slice, r, g, j]
    S = S.movedim(-2, -3).reshape(*lead, nh, ncb, dkp, 8)               # row g * rpl + r
    S = S.movedim(-3, -2).reshape(*lead, nh, dkp, ncb * 8)[..., :dk, :dv].contiguous()
    if mode != WALK_EXP_GATES:
        return S, None, None
    n = state[..., 0, dkp * 8: dkp * 8 + dkp].reshape(*lead, nh, rpl // 4, 8, 4)     # [.., h, r4, g, i]
    n = n.movedim(-2, -3).reshape(*lead, nh, dkp)[..., :dk].contiguous()
    return S, n, state[..., 0, dkp * 8 + dkp].contiguous()


def state_walk(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, heads_per_group: int, gates: Optional[torch.Tensor],
               params, cap: float, q_scale: float, mode: int, state: torch.Tensor, ctx, nh: int, dk: int, dv: int,
               segments=None, inv_freq: Optional[torch.Tensor] = None, k_scale: float = 1.0) -> torch.Tensor:
    """The recurrence S_t = a_t S_(t-1) + b_t k_t v_t^T, o_t = S_t^T q_t per head with one decay a_t and one
    input weight b_t per (token, head), token by token along every entry of the step, from and into
    state [slots, *walk_state_shape(nh, dk, dv, mode)] (float32) at the entries' state slots.  q and k of
    head h are columns q_off / k_off + (h // heads_per_group) * dk of proj [T, N], v columns v_off + h * dv;
    q is multiplied by q_scale.  ``gates`` float32 [T, M] and ``params`` (float32 [nh] each):

    * WALK_EXP_GATES: gates columns h and nh + h are the input and forget gates' pre-activations, params
      (input bias, forget bias); i = cap tanh((x + b) / cap), f = log_sigmoid(cap tanh(...)), a running
      maximum m (starting at 0) keeps the exponentials in range, a normaliser vector n moves beside S,
      and the result is o / (max(|n . q|, exp(-m)) + 1e-6);
    * WALK_STATE_SPACE: gates column h is the step size before its softplus, params (its bias, A_log, D);
      a = exp(-exp(A_log) dt), b = dt, and the result is o + D v;
    * WALK_FIXED_DECAY: no gates (``gates`` None); params (the heads' decays,): a = decay[h], b = ``k_scale``
      (the keys' scale), and, with ``inv_freq`` (float32 [r / 2]), the leading r elements of every q and k head
      are first turned by rotary positions, element i with element i + r/2 by the angle position x
      inv_freq[i], in float; the result is o.

    ``segments`` = (segs, ent_segs) on the device (see :func:`gla_segments`): long entries are then walked
    segment by segment side by side.  A stretch of tokens acts on the state as S -> D S + L (D the product of
    its decays, one number a head; L what it makes of a zero state), so every segment is first walked from
    nothing, the true start states follow one from the other, and a second walk from those writes the
    outputs (results equal to rounding).  Returns float32 [T, nh * dv]."""
    _dev(proj, gates, state, inv_freq, *params)
    T, N = proj.shape
    groups = nh // heads_per_group if heads_per_group > 0 else 0
    _need(1 <= dk <= WALK_MAX_KEY_DIM and dv >= 1 and nh >= 1 and heads_per_group >= 1 and nh % heads_per_group == 0,
          f"state_walk: key channels 1..{WALK_MAX_KEY_DIM}, heads a multiple of the heads a group")
    _need(min(q_off, k_off, v_off) >= 0 and max(q_off, k_off) + groups * dk <= N and v_off + nh * dv <= N,
          "state_walk: q, k and v columns must lie inside proj")
    _need(mode in (WALK_EXP_GATES, WALK_STATE_SPACE, WALK_FIXED_DECAY),
          "state_walk: mode 0 (exponential gates), 1 (state space) or 2 (a fixed decay per head)")
    n_par, n_cols = (2, 2 * nh) if mode == WALK_EXP_GATES else (3, nh) if mode == WALK_STATE_SPACE else (1, 0)
    rot_dim = 0
    if mode == WALK_FIXED_DECAY:
        _need(gates is None, "state_walk: a fixed decay reads no gates")
        if inv_freq is not None:
            _need(inv_freq.dtype == torch.float32 and inv_freq.dim() == 1 and 1 <= inv_freq.shape[0] <= dk // 2
                  and ctx.positions.shape == (T,), "state_walk: inv_freq float32 [r / 2], r <= dk, and the step's positions [T]")
            rot_dim = 2 * inv_freq.shape[0]
    else:
        _need(inv_freq is None and k_scale == 1.0, "state_walk: rotation and a key scale belong to the fixed-decay mode")
        _need(gates.dtype == torch.float32 and gates.dim() == 2 and gates.shape[0] == T and gates.shape[1] >= n_cols,
              f"state_walk: gates float32 [T, >= {n_cols}] wanted")
    _need(len(params) == n_par and all(p.dtype == torch.float32 and p.shape == (nh,) for p in params),
          f"state_walk: {n_par} float32 [nh] parameter vectors wanted")
    _need(state.dtype == torch.float32 and tuple(state.shape[1:]) == walk_state_shape(nh, dk, dv, mode),
          "state_walk: state must be float32 [slots, *walk_state_shape(nh, dk, dv, mode)]")
    _need(ctx.state_slots.shape == (ctx.n_entries,) and ctx.cu_tokens.shape == (ctx.n_entries + 1,) and ctx.n_tokens == T,
          "state_walk: the step's per-entry arrays do not fit")
    out = torch.empty(T, nh * dv, dtype=torch.float32, device=proj.device)
    p = list(params) + [None] * (3 - n_par)
    g_stride = gates.shape[1] if gates is not None else 0
    rot = (_ptr(ctx.positions) if rot_dim else None, _ptr(inv_freq) if rot_dim else None, rot_dim, float(k_scale))
    if segments is not None:
        segs, ent_segs = segments
        _dev(segs, ent_segs)
        _i32(segs, "segs")
        _i32(ent_segs, "ent_segs")
        n_segs = segs.numel() // 4
        _need(segs.numel() == 4 * n_segs and ent_segs.numel() == 2 * ctx.n_entries and n_segs >= ctx.n_entries,
              "state_walk: segs [n, 4] and ent_segs [entries, 2] wanted")
        shape = (n_segs,) + walk_state_shape(nh, dk, dv, mode)
        seg_local = torch.empty(shape, dtype=torch.float32, device=proj.device)
        seg_start = torch.empty(shape, dtype=torch.float32, device=proj.device)
        seg_decay = torch.empty(n_segs, nh, dtype=torch.float32, device=proj.device)
        _run("sharpi_state_walk_segmented", _ptr(proj), _code(proj.dtype), N, int(q_off), int(k_off), int(v_off),
             int(heads_per_group), _ptr(gates), g_stride, _ptr(p[0]), _ptr(p[1]), _ptr(p[2]), float(cap), float(q_scale),
             int(mode), _ptr(state), _ptr(ctx.state_slots), _ptr(ctx.cu_tokens), _ptr(out), ctx.n_entries, nh, dk, dv,
             _ptr(segs), _ptr(ent_segs), n_segs, _ptr(seg_local), _ptr(seg_start), _ptr(seg_decay), *rot, _stream())
        return out
    _run("sharpi_state_walk", _ptr(proj), _code(proj.dtype), N, int(q_off), int(k_off), int(v_off), int(heads_per_group),
         _ptr(gates), g_stride, _ptr(p[0]), _ptr(p[1]), _ptr(p[2]), float(cap), float(q_scale), int(mode), _ptr(state),
         _ptr(ctx.state_slots), _ptr(ctx.cu_tokens), _ptr(out), ctx.n_entries, nh, dk, dv, *rot, _stream())
    return out


def group_norm_gate(o: torch.Tensor, weight: Optional[torch.Tensor], eps: float, groups: int, out_dtype: torch.dtype,
                    gate_proj: Optional[torch.Tensor] = None, gate_off: int = 0, gate_act: int = GATE_NONE,
                    gate_first: bool = False) -> torch.Tensor:
    """o float32 [T, N] in `groups` equal parts, each divided by its root mean square, times weight
    (float32 [N]; None: no weight), times act(gate) (columns gate_off.. of gate_proj [T, M], of out_dtype; act GATE_SILU
    or GATE_SIGMOID_ACT).  ``gate_first``: the gate multiplies o before the statistics are taken."""
    _dev(o, weight, gate_proj)
    T, N = o.shape
    _need(o.dtype == torch.float32 and groups >= 1 and N % groups == 0
          and (weight is None or (weight.dtype == torch.float32 and weight.shape == (N,))),
          "group_norm_gate: o float32 [T, N], N a multiple of the groups, weight float32 [N] or None")
    _need(gate_act in (GATE_NONE, GATE_SILU, GATE_SIGMOID_ACT), "group_norm_gate: gate_act 0, 1 or 2")
    stride = 0
    if gate_act != GATE_NONE:
        _need(gate_proj is not None and gate_proj.dtype == out_dtype and gate_proj.dim() == 2 and gate_proj.shape[0] == T
              and 0 <= gate_off and gate_off + N <= gate_proj.shape[1], "group_norm_gate: the gate's columns must lie inside gate_proj")
        stride = gate_proj.shape[1]
    out = torch.empty(T, N, dtype=out_dtype, device=o.device)
    _run("sharpi_group_norm_gate", _ptr(o), _ptr(weight), float(eps), _ptr(gate_proj) if gate_act else None, _code(out_dtype),
         stride, int(gate_off), int(gate_act), 1 if gate_first else 0, _ptr(out), T, groups, N // groups, _stream())
    return out


def short_conv(proj: torch.Tensor, c_off: int, channels: int, weight: torch.Tensor, bias: Optional[torch.Tensor],
               tail: Optional[torch.Tensor], ctx, update_tail: bool = True) -> torch.Tensor:
    """silu(bias + causal convolution over time) on `channels` columns of proj [T, N] from c_off: weight
    float32 [channels, taps] (the last column is the current token's), bias float32 [channels] or None; tail
    float32 [slots, taps - 1, channels] carries each request's last inputs from step to step (None when
    taps is 1) and is brought up to date unless update_tail is False.  Returns [T, channels] of proj's dtype."""
    _dev(proj, weight, bias, tail)
    T, N = proj.shape
    taps = weight.shape[1] if weight.dim() == 2 else 0
    _need(weight.dtype == torch.float32 and weight.shape == (channels, taps) and 1 <= taps <= SHORT_CONV_MAX_TAPS,
          f"short_conv: weight must be float32 [channels, 1..{SHORT_CONV_MAX_TAPS} taps]")
    _need(0 <= c_off and c_off + channels <= N, "short_conv: the channels must lie inside proj")
    _need(bias is None or (bias.dtype == torch.float32 and bias.shape == (channels,)), "short_conv: bias must be float32 [channels]")
    if taps > 1:
        _need(tail is not None and tail.dtype == torch.float32 and tail.dim() == 3 and tuple(tail.shape[1:]) == (taps - 1, channels),
              "short_conv: tail must be float32 [slots, taps - 1, channels]")
    _need(ctx.state_slots.shape == (ctx.n_entries,) and ctx.cu_tokens.shape == (ctx.n_entries + 1,)
          and ctx.entry_of_token.shape == (T,), "short_conv: the step's per-entry arrays do not fit")
    out = torch.empty(T, channels, dtype=proj.dtype, device=proj.device)
    _run("sharpi_short_conv", _ptr(proj), _code(proj.dtype), N, int(c_off), _ptr(weight), _ptr(bias), taps,
         _ptr(tail) if taps > 1 else None, _ptr(ctx.state_slots), _ptr(ctx.entry_of_token), _ptr(ctx.cu_tokens), _ptr(out),
         T, ctx.n_entries, channels, 1 if update_tail else 0, _stream())
    return out


def sigmoid_gate(x: torch.Tensor, gate_proj: torch.Tensor, gate_off: int) -> torch.Tensor:
    """x [T, N] * sigmoid(gate), the gate columns gate_off.. of gate_proj [T, M] (same dtype)."""
    _dev(x, gate_proj)
    T, N = x.shape
    _need(gate_proj.dtype == x.dtype and gate_proj.dim() == 2 and gate_proj.shape[0] == T and 0 <= gate_off
          and gate_off + N <= gate_proj.shape[1], "sigmoid_gate: the gate's columns must lie inside gate_proj")
    out = torch.empty_like(x)
    _run("sharpi_sigmoid_gate", _ptr(x), _ptr(gate_proj), _code(x.dtype), gate_proj.shape[1], int(gate_off), _ptr(out), T, N, _stream())
    return out


class BranchSum:
    """Stands for a sum of branch outputs with a scale each, sum_b scales[b] * xs[b], still to be formed
    (in float): [T, N].  ``stream_add`` folds it into the residual sum; ``tensor()`` forms it alone."""

    def __init__(self, xs, scales):
        self.xs, self.scales = list(xs), [float(s) for s in scales]
        self.shape, self.dtype = tuple(xs[0].shape), torch.float32

    def tensor(self) -> torch.Tensor:
        h = torch.zeros(self.shape, dtype=torch.float32, device=self.xs[0].device)
        stream_add(h, self)
        return h


def stream_add(h: torch.Tensor, delta, out_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """h (float32 [T, N]) += delta in place, in float; delta a tensor [T, N], a BranchSum (up to 4 scaled
    branches, added in their order) or None.  With ``out_dtype`` the new h is also returned in that
    storage type."""
    import ctypes

    xs = delta.xs if isinstance(delta, BranchSum) else [] if delta is None else [delta]
    scales = delta.scales if isinstance(delta, BranchSum) else [1.0] * len(xs)
    _dev(h, *xs)
    _need(h.dim() == 2 and h.dtype == torch.float32 and len(xs) <= 4, "stream_add: h float32 [T, N], at most 4 branches")
    for x in xs:
        _need(tuple(x.shape) == tuple(h.shape) and x.dtype == xs[0].dtype, "stream_add: branches of h's shape and of one dtype")
    n = len(xs)
    out = torch.empty(h.shape, dtype=out_dtype, device=h.device) if out_dtype is not None else None
    xp = (ctypes.c_void_p * max(n, 1))(*[x.data_ptr() for x in xs])
    sp = (ctypes.c_float * max(n, 1))(*scales)
    _run("sharpi_stream_add", _ptr(h), ctypes.cast(xp, ctypes.c_void_p), ctypes.cast(sp, ctypes.c_void_p), n,
         _code(xs[0].dtype) if xs else (_code(out_dtype) if out_dtype is not None else 0), _ptr(out),
         _code(out_dtype) if out_dtype is not None else 0, h.numel(), _stream())
    return out


def side_gate(gate: torch.Tensor, ids: torch.Tensor, table: torch.Tensor, col_off: int) -> torch.Tensor:
    """gelu_tanh(gate [T, D]) * table[ids[t], col_off : col_off + D]: a slice of each token's row of a side
    table, gated element by element."""
    _dev(gate, ids, table)
    _i32(ids, "ids")
    T, D = gate.shape
    _need(ids.shape == (T,) and table.dim() == 2 and 0 <= col_off and col_off + D <= table.shape[1],
          "side_gate: ids [T]; the slice must lie inside the table's rows")
    out = torch.empty_like(gate)
    _run("sharpi_side_gate", _ptr(gate), _code(gate.dtype), _ptr(ids), _ptr(table), _code(table.dtype), table.shape[1],
         int(col_off), _ptr(out), T, D, _stream())
    return out


# ---------------------------------------------------------------------------
# several residual streams; the difference of two score maps
# ---------------------------------------------------------------------------
HYPER_MAX_STREAMS = 8                 # csrc/hyper.hip kHyperMaxStreams
HYPER_MAX_WIDTH = 15 * 1024           # floats of a row that the kernel keeps in LDS


def hyper_step(src: torch.Tensor, lanes: Optional[torch.Tensor], n_streams: int, delta=None,
               mix: Optional[torch.Tensor] = None, out_w: Optional[torch.Tensor] = None, in_w: Optional[torch.Tensor] = None,
               norm_w: Optional[torch.Tensor] = None, eps: float = 0.0, out_dtype: Optional[torch.dtype] = None,
               rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """What lies between two sublayers of a model with S residual streams per token.  ``src``: the old
    streams, float32 [T, S, W], or [T, W] when all S are still that one row.  With ``delta`` (the last
    sublayer's output [T, W], a tensor or an ExpertSum) the streams are first brought up to date,
    new[t] = sum_s mix[s, t] old[s] + out_w[t] delta (``mix`` float32 [S, S], ``out_w`` float32 [S]), and stored
    in ``lanes`` (float32 [T, S, W]; may be ``src`` itself; None: not stored).  Then u = sum_s in_w[s] new[s]
    (``in_w`` float32 [S]; None: the plain sum), and the result is unit_rms(u) * norm_w in ``out_dtype``,
    or, with ``norm_w`` None, u itself in float32.  ``rows`` (int32): only those tokens are produced."""
    lazy = delta if isinstance(delta, ExpertSum) else None
    base = lazy.y if lazy is not None else delta
    _dev(src, lanes, base, mix, out_w, in_w, norm_w, rows, *( [lazy.inv_pos, lazy.shared, lazy.weights] if lazy is not None else []))
    _i32(rows, "rows")
    S = int(n_streams)
    _need(src.dtype == torch.float32 and src.dim() in (2, 3) and 1 <= S <= HYPER_MAX_STREAMS, "hyper_step: src float32 [T, S, W] or [T, W]")
    T, W = src.shape[0], src.shape[-1]
    _need(W <= HYPER_MAX_WIDTH and (src.dim() == 2 or src.shape[1] == S), "hyper_step: streams or width do not fit")
    src_token, src_stream = (W, 0) if src.dim() == 2 else (S * W, W)
    if lanes is not None:
        _need(lanes.dtype == torch.float32 and tuple(lanes.shape) == (T, S, W), "hyper_step: lanes must be float32 [T, S, W]")
    if delta is not None:
        _need(tuple(delta.shape) == (T, W), f"hyper_step: delta {tuple(delta.shape)} vs [T, W] = {(T, W)}")
        _need(mix is not None and out_w is not None and mix.dtype == torch.float32 and mix.shape == (S, S)
              and out_w.dtype == torch.float32 and out_w.shape == (S,), "hyper_step: mix float32 [S, S] and out_w float32 [S] come with delta")
    if in_w is not None:
        _need(in_w.dtype == torch.float32 and in_w.shape == (S,), "hyper_step: in_w must be float32 [S]")
    if norm_w is not None:
        _need(norm_w.shape == (W,) and out_dtype is not None, "hyper_step: norm_w [W] and an out_dtype")
    else:
        out_dtype = torch.float32
    n_out = T if rows is None else rows.shape[0]
    out = torch.empty(n_out, W, dtype=out_dtype, device=src.device)
    _run("sharpi_hyper_step", _ptr(src), src_token, src_stream, _ptr(lanes), _ptr(base), _code(base.dtype) if base is not None else 0,
         _ptr(lazy.inv_pos) if lazy is not None else None, _ptr(lazy.shared) if lazy is not None else None,
         _ptr(lazy.weights) if lazy is not None else None, lazy.k if lazy is not None else 0, _ptr(mix), _ptr(out_w), _ptr(in_w),
         _ptr(norm_w), _code(norm_w.dtype) if norm_w is not None else 0, float(eps), _ptr(out), _code(out_dtype), _ptr(rows),
         n_out, S, W, _stream())
    return out


def map_difference(a: torch.Tensor, n_heads: int, vd: int, lam: float, eps: float, post: float,
                   gate_proj: Optional[torch.Tensor] = None, gate_off: int = 0) -> torch.Tensor:
    """a [T, n_heads * 2 * vd]: per head the outputs a1, a2 of two score maps over the same values.  Returns
    [T, n_heads * vd] = unit_rms(a1 - lam * a2) * post (the root mean square over a head's vd values, eps
    inside the root, in float), times sigmoid of column gate_off + head of gate_proj [T, M] where given
    (one gate number per head)."""
    _dev(a, gate_proj)
    T = a.shape[0]
    _need(a.dim() == 2 and a.shape[1] == n_heads * 2 * vd, "map_difference: a must be [T, n_heads * 2 * vd]")
    stride = 0
    if gate_proj is not None:
        _need(gate_proj.dtype == a.dtype and gate_proj.dim() == 2 and gate_proj.shape[0] == T and 0 <= gate_off
              and gate_off + n_heads <= gate_proj.shape[1], "map_difference: the gates' columns must lie inside gate_proj")
        stride = gate_proj.shape[1]
    out = torch.empty(T, n_heads * vd, dtype=a.dtype, device=a.device)
    _run("sharpi_map_difference", _ptr(a), _code(a.dtype), float(lam), float(eps), float(post), _ptr(gate_proj), stride,
         int(gate_off), _ptr(out), T, n_heads, vd, _stream())
    return out
