"""Fovosun on the GPU against the plain implementation (tests/plain_fovosun.py): every mechanism
alone, then the engine under every way of cutting requests into steps."""
import functools
import json
import math
import os
import random
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_fovosun as P
from tiny_fovosun import CONFIGS, SEEDS, STD_BY_SUFFIX, config

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def _rel_rows(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    got, want = got.double().cpu(), want.double().cpu()
    return (got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-30)


def _rel_rms(got: torch.Tensor, want: torch.Tensor) -> float:
    """The largest error of a row, as rms(difference) / rms(row)."""
    return float(_rel_rows(got, want).max())


# Float arithmetic against the plain model in double: a rotation's angle at position p is known to p * 2^-24, a state
# that has moved T times has drifted T roundings.  Whatever the design adds shows at 5e-3 and more when left out
# (test_what_the_design_adds_would_show_if_left_out).
FLOAT_KERNEL = 2e-5           # a row out of one kernel
FLOAT_WALK = 1e-4             # a row of the recurrence's output, and its state
FLOAT_LOGITS = 3e-4           # a row of logits, a layer's stream
FLOAT_SAME = 3e-5             # the same logits by another cut or in another batch
BF16_KERNEL = 8e-3            # a row out of one kernel that rounds its result to bfloat16


def _within_noise(err: torch.Tensor, noise: torch.Tensor, what: str) -> None:
    """`err`: per row, the engine's bfloat16 error; `noise`: per row, how far the plain model moves
    when it rounds to bfloat16 every tensor that a 16-bit engine may keep in 16 bits, and nothing of
    what the design computes in 32 bits (`_noise_rows`).  A row's limit is three times its noise (at least three
    times the median row's).  At most three rows in a hundred (or one) may exceed it, none two and a
    half times it.  The float32 runs of the same tests are the sharp ones."""
    limit = 3.0 * torch.maximum(noise, noise.median())
    over, far = int((err > limit).sum()), int((err > 2.5 * limit).sum())
    worst = int((err / limit).argmax())
    assert over <= max(1, 0.03 * err.numel()) and far == 0, \
        f"{what}: {over} of {err.numel()} rows over their limit, {far} far over; row {worst}: {float(err[worst]):.2e} (limit {float(limit[worst]):.2e})"


def _dithered(k):
    """bfloat16 rounding on a grid shifted by k / 1024 of a value: another draw of the same rounding noise."""
    f = 1.0 + k * 2.0 ** -10
    return lambda x: P.store_bf16(x * f) / f


def _noise_rows(run):
    """Per row, how far rounding alone moves a result: `run(store)` is the plain model with the tensors a 16-bit engine
    keeps in 16 bits rounded by `store`.  Where a head's output nearly cancels before it is divided by its root mean
    square, rounding is amplified tens of times in single rows, and which of two neighbouring rows is hit depends on
    the draw; so three draws on shifted grids are taken and a row's noise is the largest of them and of its two
    neighbours' (the three rows share what made the head small)."""
    exact = run(P._same)
    outs = [run(P.store_bf16), run(_dithered(1)), run(_dithered(-1))]
    many = isinstance(exact, list)
    per = []
    for i in range(len(exact) if many else 1):
        w = exact[i] if many else exact
        n = torch.stack([_rel_rows(o[i] if many else o, w) for o in outs]).max(0).values
        pad = torch.cat([n[:1], n, n[-1:]])
        per.append(torch.stack([pad[:-2], pad[1:-1], pad[2:]]).max(0).values)
    return (exact, per) if many else (exact, per[0])


class _Step:
    """What the kernels between projections and attention read of a step."""

    def __init__(self, lens, starts, slots):
        self.n_entries, self.n_tokens, self.max_entry_len = len(lens), sum(lens), max(lens)
        cu = [0]
        for n in lens:
            cu.append(cu[-1] + n)
        self.cu_tokens = torch.tensor(cu, dtype=torch.int32, device=DEV)
        self.entry_of_token = torch.tensor([e for e, n in enumerate(lens) for _ in range(n)], dtype=torch.int32, device=DEV)
        self.positions = torch.tensor([s + i for s, n in zip(starts, lens) for i in range(n)], dtype=torch.int32, device=DEV)
        self.state_slots = torch.tensor(slots, dtype=torch.int32, device=DEV)
        self.extras = {}


# five steps of three requests: one token, a few, many; a request left out of a step; pairs and singles at the end
PLAN = [[("a", 1), ("b", 40)], [("b", 1), ("c", 7), ("a", 2)], [("a", 9), ("c", 1)], [("c", 1), ("a", 2), ("b", 1)], [("b", 1)]]
TOTAL = {"a": 14, "b": 43, "c": 9}
SLOT_OF = {"a": 3, "b": 0, "c": 1}
BASE = {"a": 0, "b": 0, "c": 0}


def _over_plan(rows_of, call, base=BASE):
    """Runs `call(rows, ctx)` over PLAN, returns each request's outputs in order."""
    got = {r: [] for r in TOTAL}
    at = {r: 0 for r in TOTAL}
    for step in PLAN:
        ctx = _Step([n for _, n in step], [base[r] + at[r] for r, _ in step], [SLOT_OF[r] for r, _ in step])
        rows = torch.cat([rows_of[r][at[r]:at[r] + n] for r, n in step]).to(DEV)
        o = call(rows, ctx)
        i = 0
        for r, n in step:
            got[r].append(o[i:i + n].cpu())
            i += n
            at[r] += n
    return {r: torch.cat(v) for r, v in got.items()}


# ---------------------------------------------------------------------------
# the mechanisms alone
# ---------------------------------------------------------------------------
def _plain_retention(rows, H, dk, dv, decays, rot, first=0):
    """Outputs [T, H, dv] and the final states [H, dk, dv] of the plain recurrence on projected rows q | k | v."""
    T = rows.shape[0]
    u = rows.double()
    qk = H * dk
    q, k, v = u[:, :qk].reshape(T, H, dk), u[:, qk:2 * qk].reshape(T, H, dk), u[:, 2 * qk:2 * qk + H * dv].reshape(T, H, dv)
    pos = torch.arange(first, first + T)
    if rot:
        q, k = P.rotate_half_split(q, pos, rot[0], rot[1]), P.rotate_half_split(k, pos, rot[0], rot[1])
    k = k * dk ** -0.5
    S = torch.zeros(H, dk, dv, dtype=torch.float64)
    dec = torch.tensor(decays, dtype=torch.float64)[:, None, None]
    o = torch.zeros(T, H, dv, dtype=torch.float64)
    for t in range(T):
        S = dec * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hde,hd->he", S, q[t])
    return o, S


def _freqs(rot):
    return torch.tensor([rot[0] ** (-2.0 * i / rot[1]) for i in range(rot[1] // 2)], dtype=torch.float64).float().to(DEV) if rot else None


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, dk, dv, rot", [(2, 10, 24, (300.0, 6)), (5, 32, 40, (10000.0, 32)), (1, 136, 20, None), (3, 72, 50, (50.0, 72)),
                                            (2, 256, 16, (1e6, 64)), (4, 64, 33, (1000.0, 64))])
def test_retention_walks_every_entry_from_its_slots_state(dtype, H, dk, dv, rot):
    """A fixed decay per head (from 0.5 to 1), rotary positions on the leading elements inside the walk, the
    keys' scale, against the plain recurrence over whole sequences; requests that begin at positions 0, 1000
    and 37; states in slots 3, 0 and 1 of five."""
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(dk + dv)
    qk, vv = H * dk, H * dv
    pad = 8
    rows = {r: torch.randn(n, 2 * qk + vv + pad, generator=g).to(DT[dtype]) for r, n in TOTAL.items()}
    decays = [0.5 + 0.5 * i / max(1, H - 1) for i in range(H)]
    base = {"a": 0, "b": 1000, "c": 37}
    state = torch.zeros(5, *ops.walk_state_shape(H, dk, dv, ops.WALK_FIXED_DECAY), device=DEV)
    state[2].fill_(9.0)                                          # a slot no entry names
    dec = torch.tensor(decays, dtype=torch.float32, device=DEV)

    def call(x, ctx):
        return ops.state_walk(x, 0, qk, 2 * qk, 1, None, (dec,), 0.0, 1.0, ops.WALK_FIXED_DECAY, state, ctx, H, dk, dv,
                              inv_freq=_freqs(rot), k_scale=dk ** -0.5)

    got = _over_plan(rows, call, base)
    tol = FLOAT_WALK if dtype == "float32" else 2e-4             # (the walk reads 16-bit rows and is float from there on)
    for r in TOTAL:
        want, S = _plain_retention(rows[r].float(), H, dk, dv, decays, rot, base[r])
        assert _rel_rms(got[r], want.reshape(TOTAL[r], -1)) < tol, r
        kept, _, _ = ops.walk_state_matrices(state[SLOT_OF[r]], dk, dv, ops.WALK_FIXED_DECAY)
        assert _rel_rms(kept.reshape(H, -1), S.reshape(H, -1)) < tol, r
    assert bool((state[2] == 9.0).all()) and not bool(state[4].any())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_token_far_back_is_still_in_the_retentions_state(dtype):
    """A key 600 tokens back that the last query points at, under a decay of almost 1: without it the last
    output would be noise; the head that decays fast has forgotten it."""
    from sharpinference_amd import ops

    H, dk, dv, T = 2, 32, 16, 640
    g = torch.Generator().manual_seed(5)
    rows = torch.randn(T, 2 * H * dk + H * dv, generator=g) * 0.3
    for h in range(H):
        kk = rows[39, H * dk + h * dk: H * dk + (h + 1) * dk]
        kk *= 6.0
        rows[T - 1, h * dk:(h + 1) * dk] = kk * 4.0
    rows = rows.to(DT[dtype])
    decays = [0.9995, 0.9]
    state = torch.zeros(2, *ops.walk_state_shape(H, dk, dv, ops.WALK_FIXED_DECAY), device=DEV)
    dec = torch.tensor(decays, dtype=torch.float32, device=DEV)
    outs = []
    for cuts in ([T], [600, 39, 1]):
        state.zero_()
        o, at = [], 0
        for n in cuts:
            ctx = _Step([n], [at], [1])
            o.append(ops.state_walk(rows[at:at + n].to(DEV), 0, H * dk, 2 * H * dk, 1, None, (dec,), 0.0, 1.0, ops.WALK_FIXED_DECAY,
                                    state, ctx, H, dk, dv, k_scale=dk ** -0.5).cpu())
            at += n
        outs.append(torch.cat(o))
    want, _ = _plain_retention(rows.float(), H, dk, dv, decays, None)
    without = rows.float().clone()
    without[39] = 0.0
    gone, _ = _plain_retention(without, H, dk, dv, decays, None)
    assert _rel_rms(want[-1, 0:1], gone[-1, 0:1]) > 0.5 and _rel_rms(want[-1, 1:2], gone[-1, 1:2]) < 1e-6
    for o in outs:
        assert _rel_rms(o[-1:], want[-1:].reshape(1, -1)) < 5e-4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, dk, dv, rot", [(2, 32, 16, (100.0, 32)), (3, 72, 20, None), (1, 136, 9, (5000.0, 40))])
def test_long_entries_of_the_retention_walked_in_segments_side_by_side(dtype, H, dk, dv, rot):
    """Two entries of 700 and 300 tokens from states that are not zero: the segmented walk against the whole one."""
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(dk)
    lens, starts = [700, 300], [64, 5]
    rows = (torch.randn(sum(lens), 2 * H * dk + H * dv, generator=g) * 0.5).to(DT[dtype]).to(DEV)
    dec = torch.tensor([0.99 - 0.05 * h for h in range(H)], dtype=torch.float32, device=DEV)
    first = torch.randn(3, *ops.walk_state_shape(H, dk, dv, ops.WALK_FIXED_DECAY), generator=g).to(DEV)
    ctx = _Step(lens, starts, [2, 0])
    segs, ents = ops.gla_segments(lens, ctx.cu_tokens.cpu().numpy())
    segments = (torch.from_numpy(segs.reshape(-1)).to(DEV), torch.from_numpy(ents.reshape(-1)).to(DEV))
    res = []
    for sg in (None, segments):
        state = first.clone()
        o = ops.state_walk(rows, 0, H * dk, 2 * H * dk, 1, None, (dec,), 0.0, 1.0, ops.WALK_FIXED_DECAY, state, ctx, H, dk, dv,
                           segments=sg, inv_freq=_freqs(rot), k_scale=dk ** -0.5)
        res.append((o.cpu(), state.cpu()))
    assert _rel_rms(res[1][0], res[0][0]) < FLOAT_WALK
    assert _rel_rms(res[1][1].reshape(3, -1), res[0][1].reshape(3, -1)) < FLOAT_WALK
    assert torch.equal(res[1][1][1], first[1].cpu())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("S, W, T", [(1, 64, 5), (2, 72, 9), (3, 256, 70), (4, 128, 1), (8, 1000, 3), (5, 77, 4)])
def test_the_streams_between_two_sublayers(dtype, S, W, T):
    """The streams brought up to date from the old ones (mix indexed from, to), stored, read with weights,
    normalised; the first sublayer's streams all one row; the closing sum; rows picked out; in place."""
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(S * W)
    xs = torch.randn(T, S, W, generator=g)
    y = torch.randn(T, W, generator=g).to(DT[dtype])
    mix, out_w, in_w = torch.randn(S, S, generator=g), torch.randn(S, generator=g), torch.randn(S, generator=g)
    nw = (torch.rand(W, generator=g) + 0.5).to(DT[dtype])
    eps = 1e-5
    new = P.streams_write(xs.double().transpose(0, 1), y.double(), mix.double(), out_w.double())       # [S, T, W]
    want = P.rms_norm(P.streams_read(new, in_w.double()), nw.double(), eps)
    lanes = xs.clone().to(DEV)
    got = ops.hyper_step(lanes, lanes, S, y.to(DEV), mix.to(DEV), out_w.to(DEV), in_w.to(DEV), nw.to(DEV), eps, DT[dtype])
    tol = FLOAT_KERNEL if dtype == "float32" else BF16_KERNEL
    assert _rel_rms(got, want) < tol
    assert _rel_rms(lanes.reshape(T, -1), new.transpose(0, 1).reshape(T, -1)) < FLOAT_KERNEL
    # nothing waits: the streams stay, the read alone
    kept = xs.clone().to(DEV)
    got = ops.hyper_step(kept, kept, S, None, None, None, in_w.to(DEV), nw.to(DEV), eps, DT[dtype])
    assert torch.equal(kept.cpu(), xs)
    assert _rel_rms(got, P.rms_norm(P.streams_read(xs.double().transpose(0, 1), in_w.double()), nw.double(), eps)) < tol
    # the first sublayer: every stream is the one row
    h = torch.randn(T, W, generator=g).to(DEV)
    lanes = torch.full((T, S, W), 7.0, device=DEV)
    got = ops.hyper_step(h, lanes, S, None, None, None, in_w.to(DEV), nw.to(DEV), eps, DT[dtype])
    assert torch.equal(lanes, h[:, None, :].expand(T, S, W))
    assert _rel_rms(got, P.rms_norm(h.double().cpu() * float(in_w.double().sum()), nw.double(), eps)) < tol
    # the closing sum with the last output folded in, for two rows picked out
    rows = torch.tensor([T - 1, 0], dtype=torch.int32, device=DEV)
    got = ops.hyper_step(xs.to(DEV), None, S, y.to(DEV), mix.to(DEV), out_w.to(DEV), rows=rows)
    assert got.dtype == torch.float32 and _rel_rms(got, new.sum(0)[[T - 1, 0]]) < FLOAT_KERNEL


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_streams_take_a_sum_of_experts_that_is_still_to_be_formed(dtype):
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(8)
    T, S, W, k = 6, 3, 64, 2
    xs = torch.randn(T, S, W, generator=g).to(DEV)
    y = torch.randn(T * k, W, generator=g).to(DT[dtype]).to(DEV)
    shared = torch.randn(T, W, generator=g).to(DT[dtype]).to(DEV)
    wts = torch.rand(T, k, generator=g).to(DEV)
    inv = torch.randperm(T * k, generator=g).to(torch.int32).to(DEV)
    mix, out_w, in_w = torch.randn(S, S, generator=g).to(DEV), torch.randn(S, generator=g).to(DEV), torch.randn(S, generator=g).to(DEV)
    nw = torch.ones(W, dtype=DT[dtype], device=DEV)
    lazy = ops.ExpertSum(y, inv, shared, T, k, wts)
    a_l, b_l = xs.clone(), xs.clone()
    a = ops.hyper_step(a_l, a_l, S, lazy, mix, out_w, in_w, nw, 1e-6, DT[dtype])
    b = ops.hyper_step(b_l, b_l, S, lazy.tensor(), mix, out_w, in_w, nw, 1e-6, DT[dtype])
    assert torch.equal(a, b) and torch.equal(a_l, b_l)            # the bits of the combine kernel and the plain form in a row


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T, H, e, gate", [(1, 5, 80, True), (19, 3, 20, False), (70, 8, 128, True), (5, 2, 6, True), (33, 6, 64, False)])
def test_the_difference_of_two_maps_normed_and_gated_per_head(dtype, T, H, e, gate):
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(T + e)
    a = torch.randn(T, H, 2, e, generator=g).to(DT[dtype])
    proj = torch.randn(T, 11 + H, generator=g).to(DT[dtype])
    lam, diff, eps = 0.62, 0.3, 1e-5
    want = P.difference_of_maps(a[:, :, 0].double(), a[:, :, 1].double(), lam, diff, eps)
    if gate:
        want = want * torch.sigmoid(proj[:, 11:].double())[:, :, None]
    got = ops.map_difference(a.reshape(T, -1).to(DEV), H, e, lam, eps, 1.0 - diff, proj.to(DEV) if gate else None, 11)
    assert _rel_rms(got, want.reshape(T, -1)) < (FLOAT_KERNEL if dtype == "float32" else BF16_KERNEL)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, G, d, e, rot, taps, bias, temp", [
    (4, 2, 12, 20, (5000.0, 8), 0, True, None), (6, 1, 8, 6, None, 2, False, (16.0, 0.4)), (4, 2, 32, 64, None, 4, False, (32.0, 0.25)),
    (8, 2, 32, 64, (20000.0, 32), 0, True, None), (2, 2, 24, 40, None, 8, False, None), (3, 3, 10, 33, None, 0, True, (7.0, 1.5))])
def test_maps_rotated_each_on_its_own_and_queries_expanded(dtype, H, G, d, e, rot, taps, bias, temp):
    """Between the projections and attention of a differential layer: biases, the convolution with its carried
    tail, rotation of each map's own leading elements, the query temperature; key rows of both maps in the cache,
    one query row per (head, map) with zeros in the other map's place."""
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(H * d + e)
    qn, kn, vn = H * 2 * d, G * 2 * d, G * e
    C = qn + kn + vn
    rows = {r: (torch.randn(n, C + 5, generator=g)).to(DT[dtype]) for r, n in TOTAL.items()}
    b = torch.randn(C, generator=g) if bias else None
    cw = torch.randn(C, taps, generator=g) * 0.6 if taps else None
    base = {"a": 0, "b": 1000, "c": 37}
    ps = 16
    pages = {r: [] for r in TOTAL}
    free = list(torch.randperm(12, generator=g).tolist())
    for r, n in TOTAL.items():
        pages[r] = [free.pop() for _ in range((n + ps - 1) // ps)]
    kc = torch.zeros(12, G, ps, 2 * d, dtype=DT[dtype], device=DEV)
    vc = torch.zeros(12, G, e, ps, dtype=DT[dtype], device=DEV)
    tail = torch.zeros(5, max(taps - 1, 1), C, device=DEV) if taps else None
    seen = {r: 0 for r in TOTAL}

    def call(x, ctx):
        slots = []
        for ent, r in enumerate(ctx.reqs):
            for i in range(ctx.lens[ent]):
                p = seen[r] + i
                slots.append(pages[r][p // ps] * ps + p % ps)
            seen[r] += ctx.lens[ent]
        sm = torch.tensor(slots, dtype=torch.int32, device=DEV)
        return ops.qk_prep(x, 0, qn, qn + kn, H, G, 2 * d, e, ctx, kc, vc, sm, inv_freq=_freqs(rot), pair_layout=ops.PAIRS_HALF_SPLIT,
                           conv_w=cw.to(DEV) if taps else None, tail=tail, bias=b.to(DEV) if bias else None, temperature=temp, maps=2)

    got = {r: [] for r in TOTAL}
    at = {r: 0 for r in TOTAL}
    for step in PLAN:
        ctx = _Step([n for _, n in step], [base[r] + at[r] for r, _ in step], [SLOT_OF[r] for r, _ in step])
        ctx.reqs, ctx.lens = [r for r, _ in step], [n for _, n in step]
        x = torch.cat([rows[r][at[r]:at[r] + n] for r, n in step]).to(DEV)
        o = call(x, ctx).cpu()
        i = 0
        for r, n in step:
            got[r].append(o[i:i + n])
            i += n
            at[r] += n
    tol = FLOAT_KERNEL if dtype == "float32" else BF16_KERNEL
    for r, n in TOTAL.items():
        u = rows[r][:, :C].double()
        if bias:
            u = u + b.double()
        if taps:
            u = P.causal_conv(u, cw.double())
        pos = torch.arange(base[r], base[r] + n)
        q, k, v = u[:, :qn].reshape(n, H * 2, d), u[:, qn:qn + kn].reshape(n, G * 2, d), u[:, qn + kn:].reshape(n, G, e)
        if rot:
            q, k = P.rotate_half_split(q, pos, rot[0], rot[1]), P.rotate_half_split(k, pos, rot[0], rot[1])
        if temp:
            q = q * P.query_temperature(pos, temp[1], temp[0], torch.float64)[:, None, None]
        wide = torch.zeros(n, H, 2, 2, d, dtype=torch.float64)                 # [token, head, map, place, d]
        qq = q.reshape(n, H, 2, d)
        wide[:, :, 0, 0], wide[:, :, 1, 1] = qq[:, :, 0], qq[:, :, 1]
        gq = torch.cat(got[r])
        assert _rel_rms(gq, wide.reshape(n, -1)) < tol, r
        assert not bool(gq.reshape(n, H, 2, 2, d)[:, :, 0, 1].any()) and not bool(gq.reshape(n, H, 2, 2, d)[:, :, 1, 0].any())
        gk = torch.stack([kc[pages[r][p // ps], :, p % ps] for p in range(n)]).cpu()
        gv = torch.stack([vc[pages[r][p // ps], :, :, p % ps] for p in range(n)]).cpu()
        assert _rel_rms(gk.reshape(n, -1), k.reshape(n, -1)) < tol, r
        assert _rel_rms(gv.reshape(n, -1), v.reshape(n, -1)) < tol, r


class _Ctx:
    """What the attention op reads of a step of one request: `tiles` cuts its tokens into prompt
    tiles, `singles` lists them one by one."""

    def __init__(self, positions, tiles=False, singles=False, tile_tokens=64):
        T = positions.shape[0]
        self.entry_of_token, self.positions = torch.zeros(T, dtype=torch.int32, device=DEV), positions.to(DEV)
        self.n_decode, self.decode_tokens, self.n_prefill_tiles, self.prefill_tiles = 0, None, 0, None
        self.prefill_tile_tokens = tile_tokens
        if tiles:
            t = [(0, o, min(tile_tokens, T - o)) for o in range(0, T, tile_tokens)]
            self.prefill_tiles = torch.tensor(t, dtype=torch.int32, device=DEV)
            self.n_prefill_tiles = len(t)
        if singles:
            self.n_decode = T


class _Group:
    def __init__(self, bt, max_context=0):
        self.block_table, self.max_context = bt.to(DEV), max_context


def _paged(k, v, dtype, seed):
    """Keys [S, G, d] and values [S, G, e] of one request on shuffled pages of 16."""
    S, G, d = k.shape
    e = v.shape[2]
    ps = 16
    n_blocks = (S + ps - 1) // ps
    perm = torch.randperm(n_blocks + 3, generator=torch.Generator().manual_seed(seed))[:n_blocks]
    kc = torch.zeros(n_blocks + 3, G, ps, d, dtype=DT[dtype])
    vc = torch.zeros(n_blocks + 3, G, e, ps, dtype=DT[dtype])
    for p in range(S):
        kc[perm[p // ps], :, p % ps] = k[p].to(DT[dtype])
        vc[perm[p // ps], :, :, p % ps] = v[p].to(DT[dtype])
    bt = torch.full((1, n_blocks + 2), -1, dtype=torch.int32)
    bt[0, :n_blocks] = perm.to(torch.int32)
    return kc.to(DEV), vc.to(DEV), bt


KERNELS = [("float32", "float", "all"), ("bfloat16", "float", "all"), ("bfloat16", "matrix cores", "tiles"),
           ("bfloat16", "matrix cores", "singles")]


@pytest.mark.parametrize("dtype, kernel, how", KERNELS)
@pytest.mark.parametrize("window", [None, 130, 48])
@pytest.mark.parametrize("back", ["at the edge", "past the edge", "far", "a page border", "itself"])
def test_one_key_stands_out_in_one_map_only(dtype, kernel, how, window, back):
    """Differential attention over 691 positions through the attention kernels the layers use: the last
    query's second map points at one key whose value is large (scores sharpened so that it carries the
    map), the first map sees noise.  The key lies just inside the window, just outside it (it must then
    not show), far back, at a page's first place, or is the query's own."""
    from sharpinference_amd import ops

    S, H, G, d, e = 691, 4, 2, 32, 64
    first_seen = 0 if window is None else S - window
    marked = {"at the edge": first_seen, "past the edge": first_seen - 1, "far": 3, "a page border": 640, "itself": S - 1}[back]
    if marked < 0:
        pytest.skip("nothing lies before the first key")
    g = torch.Generator().manual_seed(7)
    q, k, v = torch.randn(S, H, 2, d, generator=g), torch.randn(S, G, 2, d, generator=g), torch.randn(S, G, e, generator=g)
    for h in range(H):
        kk = k[marked, h // (H // G), 1]
        q[S - 1, h, 1] = kk * (40.0 / kk.pow(2).sum())
    v[marked] *= 8.0
    q, k, v = q.to(DT[dtype]), k.to(DT[dtype]), v.to(DT[dtype])
    scale, lam, diff, eps = 1.3 / math.sqrt(d), 0.55, 0.3, 1e-6
    mask = P.visible(S, window)
    a1 = P.softmax_attention(q[:, :, 0].double(), k[:, :, 0].double(), v.double(), scale, mask)
    a2 = P.softmax_attention(q[:, :, 1].double(), k[:, :, 1].double(), v.double(), scale, mask)
    want = P.difference_of_maps(a1, a2, lam, diff, eps).reshape(S, -1)
    wide = torch.zeros(S, H, 2, 2, d, dtype=DT[dtype])
    wide[:, :, 0, 0], wide[:, :, 1, 1] = q[:, :, 0], q[:, :, 1]
    kc, vc, bt = _paged(k.reshape(S, G, 2 * d), v, dtype, seed=S)
    positions = torch.arange(S, dtype=torch.int32)
    kind = WINDOW_SLIDING if window else WINDOW_NONE
    qx = wide.reshape(S, -1).to(DEV)
    if how == "all":
        o = ops.attention_generic(qx, kc, vc, bt.to(DEV), torch.zeros(S, dtype=torch.int32, device=DEV), positions.to(DEV), kind,
                                  window or 0, scale, 2 * H, G, 2 * d, e)
    else:
        assert ops.decode_attention_ok(qx.dtype, 2 * d) and ops.prefill_attention_ok(qx.dtype, 2 * d)
        ctx = _Ctx(positions, tiles=how == "tiles", singles=how == "singles")
        o = ops.attention(qx, kc, vc, _Group(bt, S), ctx, kind, window or 0, scale, 2 * H, G, 2 * d, e)
    got = ops.map_difference(o, H, e, lam, eps, 1.0 - diff)
    err = _rel_rows(got, want)
    assert float(err[-1]) < (5e-5 if dtype == "float32" else 2e-2), f"the last row: {float(err[-1]):.2e}"
    assert float(err.max()) < (5e-5 if dtype == "float32" else 3e-2)
    # the marked key shows in the last row exactly when it is visible
    vv = v.double().clone()
    vv[marked] = 0.0
    b2 = P.softmax_attention(q[:, :, 1].double(), k[:, :, 1].double(), vv, scale, mask)
    shows = _rel_rms(a2[-1:].reshape(1, -1), b2[-1:].reshape(1, -1)) > 0.5
    assert shows == (marked >= first_seen)


from sharpinference_amd.cache.spec import WINDOW_NONE, WINDOW_SLIDING  # noqa: E402


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T, E, k, W", [(1, 12, 2, 192), (9, 5, 3, 72), (70, 4, 1, 128), (130, 3, 3, 96)])
def test_the_router_adds_its_bias_and_weighs_its_picks_by_their_own_softmax(dtype, T, E, k, W):
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(T + E)
    x = torch.randn(T, W, generator=g).to(DT[dtype])
    wr = (torch.randn(E, W, generator=g) * 0.2).to(DT[dtype])
    b = torch.randn(E, generator=g) * 2.0
    ids, wts, logits = ops.router_topk(x.to(DEV), wr.to(DEV), k, ops.GATE_SOFTMAX_PICKED, False, want_gates=True, bias=b.to(DEV))
    z = x.double() @ wr.double().T + b.double()
    assert _rel_rms(logits, z) < 1e-5
    zz = logits.double().cpu()                                     # the picks are checked on the logits the kernel saw
    val, idx = torch.topk(zz, k, dim=-1)
    assert torch.equal(ids.cpu().long(), idx)
    assert torch.allclose(wts.double().cpu(), torch.softmax(val, dim=-1), atol=1e-6)
    assert not torch.equal(idx, torch.topk(zz - b.double(), k, dim=-1)[1]) or T == 1     # the bias moves picks


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("limit", [0.7, 1.5, 7.0])
def test_the_clamped_unit_alone_and_in_the_products_epilogues(dtype, limit):
    """g = min(g, limit), u = clamp(u, -limit, limit), g sigmoid(1.702 g) (u + 1): the activation kernel against the
    plain formula on values far beyond the limit, and (bfloat16) the two grouped products that apply it in
    their epilogue against the product followed by the kernel, bit for bit."""
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(int(limit * 10))
    M, I = 37, 64
    gu = (torch.randn(M, 2 * I, generator=g) * 3.0).to(DT[dtype])
    act = ops.gated_activation("swish_clamp", limit)
    got = ops.gated_act(gu.to(DEV), None, act)
    gg, uu = gu[:, :I].double().clamp(max=limit), gu[:, I:].double().clamp(min=-limit, max=limit)
    want = gg * torch.sigmoid(1.702 * gg) * (uu + 1.0)
    assert _rel_rms(got, want) < (FLOAT_KERNEL if dtype == "float32" else BF16_KERNEL)
    if dtype != "bfloat16":
        return
    E, K, N, k = 4, 128, 128, 2
    w = (torch.randn(E, N, K, generator=g) * 0.3).to(torch.bfloat16).to(DEV)
    for T in (5, 200):                                            # the few-rows product, the many-rows product
        x = torch.randn(T, K, generator=g).to(torch.bfloat16).to(DEV)
        wr = torch.randn(E, K, generator=g).to(torch.bfloat16).to(DEV)
        ids, wts, rt = ops.route(x, wr, k, ops.GATE_SOFTMAX_PICKED)
        fused = ops.grouped_swiglu(x, w, rt, torch.bfloat16, scaled=False, act=act)
        apart = ops.gated_act(ops.grouped_linear(x, w, rt, True, torch.bfloat16), None, act)
        assert torch.equal(fused, apart)
    if ops.picked_ok(5, k, N, K, True, False):
        x = torch.randn(5, K, generator=g).to(torch.bfloat16).to(DEV)
        ids, wts = ops.router_topk(x, wr, k, ops.GATE_SOFTMAX_PICKED)
        picked = ops.gemm_skinny_picked(x, w, ids, None, False, True, act, torch.bfloat16)
        rows = torch.stack([x[t] for t in range(5) for _ in range(k)])
        ref = torch.stack([(rows[i].float() @ w[int(ids.reshape(-1)[i])].float().T) for i in range(5 * k)]).to(torch.bfloat16)
        assert _rel_rms(picked, ops.gated_act(ref, None, act)) < 2e-2


# ---------------------------------------------------------------------------
# the engine
# ---------------------------------------------------------------------------
@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    from sharpinference_amd import load_config
    from sharpinference_amd.weights.loader import write_random_model

    out = {}
    for name in CONFIGS:
        d = str(tmp_path_factory.mktemp("fovosun_" + name))
        write_random_model(load_config(config(name)), d, SEEDS[name], std=0.1, std_by_suffix=STD_BY_SUFFIX)
        out[name] = d
    return out


@functools.lru_cache(maxsize=8)
def _plain_model(d):
    return P.read_config(d), P.load_weights(d, torch.float64)


def _engine(d, dtype, **kw):
    from sharpinference_amd.engine import Engine

    args = dict(dtype=dtype, device=DEV, max_num_seqs=4, kv_tokens=1024, max_model_len=1024)
    args.update(kw)
    return Engine(d, **args)


def _run(eng, reqs, steps, free=True, picks=None):
    """steps: lists of (request id, number of its next tokens).  Returns per request the logits at
    every position.  ``picks`` (a dict) receives per request, for every routed layer in order, the
    experts and weights the engine's router chose at every position."""
    from sharpinference_amd.engine import StepEntry

    at = {r: 0 for r in reqs}
    logits = {r: [] for r in reqs}
    chosen = {r: [] for r in reqs}
    for step in steps:
        entries = []
        for r, n in step:
            if at[r] == 0:
                eng.add_request(r)
            entries.append(StepEntry(r, reqs[r][at[r]:at[r] + n], list(range(n))))
        trace = [] if picks is not None else None
        out = eng.step(entries, router_trace=trace).cpu()
        o = 0
        for r, n in step:
            logits[r].append(out[o:o + n])
            if trace is not None:
                chosen[r].append([(ids[o:o + n].cpu().long(), wts[o:o + n].cpu().double()) for ids, wts, _ in trace])
            o += n
            at[r] += n
            if at[r] == len(reqs[r]) and free:
                eng.free_request(r)
    if picks is not None:
        for r, parts in chosen.items():
            picks[r] = [(torch.cat([p[l][0] for p in parts]), torch.cat([p[l][1] for p in parts])) for l in range(len(parts[0]))]
    return {r: torch.cat(v) for r, v in logits.items()}


@functools.lru_cache(maxsize=64)
def _plain_logits(d, toks, rounded=False):
    cfg, w = _plain_model(d)
    return P.forward(cfg, w, list(toks), store=P.store_bf16 if rounded else P._same)


def _check(d, dtype, reqs, got, what, picks=None):
    """float32: against the plain model with its own router.  bfloat16: against the plain model run with the
    experts the engine picked (a close call between two experts' logits falls either way once the rows are
    rounded; the picks themselves are pinned by the float32 runs and the router's own test)."""
    for r, toks in reqs.items():
        if dtype == "float32":
            err = _rel_rows(got[r], _plain_logits(d, tuple(toks)))
            assert float(err.max()) < FLOAT_LOGITS, f"{what}, request {r}: {float(err.max()):.2e} at row {int(err.argmax())}"
        else:
            cfg, w = _plain_model(d)
            want, noise = _noise_rows(lambda store: P.forward(cfg, w, list(toks), router_picks=picks[r] if picks else None, store=store))
            _within_noise(_rel_rows(got[r], want), noise, f"{what}, request {r}")


def _run_and_check(eng, d, dtype, reqs, steps, what):
    picks = {} if dtype == "bfloat16" else None
    got = _run(eng, reqs, steps, picks=picks)
    _check(d, dtype, reqs, got, what, picks)
    return got


def _tokens(n, vocab, seed):
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


def _cuts(total, sizes):
    out, i = [], 0
    while total > 0:
        n = min(total, sizes[i % len(sizes)])
        out.append(n)
        total -= n
        i += 1
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_every_layers_streams_agree_with_the_plain_model(model_dirs, name, dtype):
    """The sum of the residual streams after every layer of a 40-token prompt, in float as the engine keeps them."""
    from sharpinference_amd import ops
    from sharpinference_amd.engine import StepEntry

    d = model_dirs[name]
    cfg, w = _plain_model(d)
    toks = _tokens(40, CONFIGS[name]["vocab"], 9)
    eng = _engine(d, dtype)
    caught = []
    for b in eng.model.blocks:
        def fwd(stream, ctx, cache, orig=b.forward):
            orig(stream, ctx, cache)
            if stream.lanes is not None:
                assert stream.lanes.dtype == torch.float32
                mix, out_w = stream.pending_lanes
                caught.append(ops.hyper_step(stream.lanes, None, stream.lanes.shape[1], stream.pending, mix, out_w).clone())
            else:
                caught.append((stream.h + stream.pending_tensor().float()).clone())
        b.forward = fwd
    eng.add_request("x")
    trace = []
    eng.step([StepEntry("x", toks, [39])], router_trace=trace)
    eng.free_request("x")
    picks = [(ids.cpu().long(), wts.cpu().double()) for ids, wts, _ in trace] if dtype == "bfloat16" else None
    def layers(store):
        out = []
        P.forward(cfg, w, toks, layer_outputs=out, store=store, router_picks=picks)
        return out
    if dtype == "float32":
        want, noise = layers(P._same), None
    else:
        want, noise = _noise_rows(layers)
    assert len(caught) == len(want)
    for i, (a, b) in enumerate(zip(caught, want)):
        if dtype == "float32":
            assert _rel_rms(a, b) < FLOAT_LOGITS, f"layer {i}: {_rel_rms(a, b):.2e}"
        else:
            _within_noise(_rel_rows(a, b), noise[i], f"layer {i}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompts_portions_and_decoding_agree_with_the_plain_model(model_dirs, name, dtype):
    d = model_dirs[name]
    vocab = CONFIGS[name]["vocab"]
    eng = _engine(d, dtype)
    toks = _tokens(150, vocab, 1)
    ways = {
        "whole": [150],
        "decoded one by one": [1] * 3 + [99] + [1] * 48,          # the first tokens alone, then a tail through page borders and windows
        "portions": _cuts(150, [2, 3, 17, 2, 64, 5, 16, 1, 31]),
        "pairs": [2] * 75,
    }
    first = None
    for what, cuts in ways.items():
        got = _run_and_check(eng, d, dtype, {what: toks}, [[(what, n)] for n in cuts], f"{name} {dtype} {what}")
        if dtype == "float32":
            first = got[what] if first is None else first
            assert _rel_rms(got[what], first) < FLOAT_SAME, f"{what}: the cut changes the logits"
    assert eng.runner.graph_replays > 0                           # decode steps ran from graphs, states and all
    eng.cache.check_invariants()
    assert not eng.cache.requests


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["odd", "even"])
def test_a_long_prompt_agrees_with_its_portions(model_dirs, name, dtype):
    """700 tokens in one step (the retention's segments side by side) and in portions of 100: far keys, windows that
    have long passed, states that have moved hundreds of times."""
    d = model_dirs[name]
    toks = _tokens(700, CONFIGS[name]["vocab"], 8)
    eng = _engine(d, dtype, kv_tokens=2048)
    whole = _run_and_check(eng, d, dtype, {"w": toks}, [[("w", 700)]], f"{name} {dtype} 700 tokens at once")
    parts = _run_and_check(eng, d, dtype, {"p": toks}, [[("p", 100)] for _ in range(7)], f"{name} {dtype} 700 tokens in portions")
    if dtype == "float32":
        assert _rel_rms(whole["w"], parts["p"]) < FLOAT_SAME


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_first_tokens_and_a_long_decoded_tail(model_dirs, dtype):
    """Every token from the first decoded alone: 260 steps (the convolutions' tails and the states start from
    zeros, the windows pass over decoded tokens), replayed from graphs."""
    d = model_dirs["odd"]
    toks = _tokens(260, CONFIGS["odd"]["vocab"], 7)
    eng = _engine(d, dtype)
    _run_and_check(eng, d, dtype, {"x": toks}, [[("x", 1)] for _ in toks], f"decoded from the first token, {dtype}")
    assert eng.runner.graph_replays >= 250
    assert all(g.pool.num_free == g.pool.num_pages for g in eng.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["odd", "even", "wide"])
def test_unequal_requests_in_one_batch_give_what_each_gives_alone(model_dirs, name, dtype):
    d = model_dirs[name]
    vocab = CONFIGS[name]["vocab"]
    reqs = {"a": _tokens(90, vocab, 2), "b": _tokens(37, vocab, 3), "c": _tokens(130, vocab, 4), "d": _tokens(5, vocab, 5)}
    steps = [[("a", 29), ("b", 2)], [("a", 1), ("b", 33), ("c", 64)], [("c", 2), ("a", 1), ("d", 5), ("b", 1)],
             [("a", 59), ("c", 1), ("b", 1)], [("c", 63)]]
    eng = _engine(d, dtype)
    got = _run_and_check(eng, d, dtype, reqs, steps, f"mixed {dtype}")
    if dtype == "float32":
        for r, toks in reqs.items():
            alone = _run(eng, {r: toks}, [[(r, len(toks))]])
            assert _rel_rms(got[r], alone[r]) < FLOAT_SAME, f"{r}: the batch changes the logits"
    eng.cache.check_invariants()


def test_pages_and_slots_are_given_back_and_used_again(model_dirs):
    """Two state slots and a pool of a dozen pages serve ten requests in turn: a state or a tail that a request
    before left in its slot, or a key in a page used again, would show."""
    d = model_dirs["even"]
    vocab = CONFIGS["even"]["vocab"]
    eng = _engine(d, "float32", max_num_seqs=2, kv_tokens=192, max_model_len=160, max_tokens_per_step=64)
    slots = set()
    for i in range(5):
        a, b = f"a{i}", f"b{i}"
        reqs = {a: _tokens(100 + i, vocab, 10 + i), b: _tokens(60 - i, vocab, 20 + i)}
        steps = [[(a, 40), (b, 3)], [(a, 60 + i), (b, 57 - i - 1)], [(b, 1)]]
        eng.add_request(a), eng.add_request(b)
        slots |= {eng.cache.requests[a].state_slot, eng.cache.requests[b].state_slot}
        eng.free_request(a), eng.free_request(b)
        got = _run(eng, reqs, steps)
        _check(d, "float32", reqs, got, f"round {i}")
        eng.cache.check_invariants()
    for g in eng.cache.groups:
        assert g.pool.total_allocs > 2 * g.pool.num_pages and g.pool.num_free == g.pool.num_pages
    assert len(slots) == 2


def test_what_the_design_adds_would_show_if_left_out(model_dirs):
    """The weights of these tests make each mechanism matter: the plain model without it is far
    from the engine, the plain model with it is not."""
    d = model_dirs["odd"]
    cfg, w = _plain_model(d)
    toks = _tokens(80, CONFIGS["odd"]["vocab"], 6)
    eng = _engine(d, "float32")
    got = _run(eng, {"x": toks}, [[("x", 50)], [("x", 30)]])["x"]
    assert _rel_rms(got, P.forward(cfg, w, toks)) < FLOAT_LOGITS

    def changed(what):
        c = json.loads(json.dumps(cfg))
        ww = dict(w)

        def each(suffix, f):
            for k in w:
                if k.endswith(suffix):
                    ww[k] = f(w[k])

        def mixers(kind):
            return [l["mixer"] for l in c["layers"] if l["type"] in kind]
        if what == "one map alone":
            for m in mixers(("attention", "attention_2")):
                m["diff"] = 0.0
            each(".lq1", lambda t: torch.full_like(t, -9.0)), each(".lk1", lambda t: torch.full_like(t, 9.0))
            each(".lq2", lambda t: torch.full_like(t, -9.0)), each(".lk2", lambda t: torch.full_like(t, 9.0))
        elif what == "lambda its constant alone":
            each(".lq1", torch.zeros_like), each(".lq2", torch.zeros_like)
        elif what == "no window":
            for m in mixers(("attention_2",)):
                m.pop("mask", None)
        elif what == "a window one token wider":
            for m in mixers(("attention_2",)):
                if "mask" in m:
                    m["mask"]["size"] += 1
        elif what == "no rotation":
            for m in mixers(("attention_2", "retention")):
                m.pop("rot", None)
        elif what == "the whole head rotated as one":
            for m in mixers(("attention_2",)):
                if "rot" in m:
                    m["rot"]["base"] *= 3.0
        elif what == "no query temperature":
            for m in mixers(("attention",)):
                m.pop("q_temp", None)
        elif what == "a convolution of the current token alone":
            def ident(t):
                o = torch.zeros_like(t)
                o[:, -1] = 1.0
                return o
            each(".conv", ident)
        elif what == "no biases":
            for k in w:
                if ".mix." in k and k.endswith(".b"):
                    ww[k] = torch.zeros_like(w[k])
        elif what == "no head gate":
            for k in w:
                if k.endswith("mix.g") and w[k].shape[0] < 16:
                    ww[k] = torch.zeros_like(w[k])
        elif what == "decays exchanged":
            for m in mixers(("retention",)):
                m["decay"] = m["decay"][::-1]
        elif what == "no router bias":
            each("router.b", torch.zeros_like)
        elif what == "another limit":
            for l in c["layers"]:
                if l["mlp"] and l["mlp"]["kind"] == "dense":
                    l["mlp"]["limit"] *= 0.5
                elif l["mlp"]:
                    l["mlp"]["expert"]["limit"] *= 0.5
        elif what == "the shared expert with the experts' limit":
            for l in c["layers"]:
                if l["mlp"] and l["mlp"].get("shared"):
                    l["mlp"]["shared"]["limit"] = l["mlp"]["expert"]["limit"]
        elif what == "streams mixed the other way round":
            each(".mix", lambda t: t.T.contiguous())
        elif what == "every stream read alike":
            each(".in", lambda t: torch.full_like(t, float(t.mean())))
        elif what == "no embedding scale":
            c["embedding"]["scale"] = 1.0
        return float(_rel_rows(got, P.forward(c, ww, toks)).max())

    for what in ("one map alone", "lambda its constant alone", "no window", "a window one token wider", "no rotation",
                 "the whole head rotated as one", "no query temperature", "a convolution of the current token alone", "no biases",
                 "no head gate", "decays exchanged", "no router bias", "another limit", "the shared expert with the experts' limit",
                 "streams mixed the other way round", "every stream read alike", "no embedding scale"):
        assert changed(what) > 5e-3, what


@pytest.mark.parametrize("name", list(CONFIGS))
def test_greedy_generation_through_the_scheduler(model_dirs, name):
    d = model_dirs[name]
    cfg, w = _plain_model(d)
    vocab = CONFIGS[name]["vocab"]
    prompts = [_tokens(n, vocab, 30 + n) for n in (5, 41, 18)]
    want = [P.generate(cfg, w, p, 8) for p in prompts]
    eng = _engine(d, "float32", max_tokens_per_step=16)          # prompts are cut into portions beside decode tokens
    got = [r.token_ids for r in eng.generate(prompts, max_new_tokens=8, temperature=0.0)]
    assert got == want
    eng.cache.check_invariants()
    assert not eng.cache.requests and eng.last_stats.steps > 8


def test_the_command_line_generates_from_this_design(model_dirs):
    d = model_dirs["odd"]
    cfg, w = _plain_model(d)
    prompt = _tokens(12, CONFIGS["odd"]["vocab"], 77)
    want = P.generate(cfg, w, prompt, 6)
    cmd = [sys.executable, os.path.join(ROOT, "bin", "sharpi-cli"), "-m", d, "--prompt-ids", " ".join(map(str, prompt)), "-n", "6",
           "--temp", "0", "--dtype", "fp32", "--repeat-penalty", "1.0", "--no-display-prompt", "--ignore-eos", "--ctx-size", "256"]
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=110)
    assert out.returncode == 0, out.stderr[-2000:]
    assert [int(t) for t in out.stdout.split() if t.lstrip("-").isdigit()][:6] == want, out.stdout


def test_the_trace_runner_replays_this_design(model_dirs, tmp_path):
    d = model_dirs["odd"]
    cfg, w = _plain_model(d)
    vocab = CONFIGS["odd"]["vocab"]
    a, b = _tokens(70, vocab, 41), _tokens(20, vocab, 42)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:33], "want": [0, 32]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[33:35], "want": []}, {"id": "b", "tokens": b, "want": [19]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[35:69], "want": [33]}], "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": a[69:], "want": [0]}], "end": ["a"]}]
    out = str(tmp_path / "out")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", "float32", "--out", out,
           "--max-tokens", "128"]
    p = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    for st in steps:
        p.stdin.write(json.dumps(st) + "\n")
        p.stdin.flush()
        assert p.stdout.readline().strip() == f"done {st['step']}"
    p.stdin.close()
    assert p.wait(timeout=60) == 0
    wa, wb = P.forward(cfg, w, a), P.forward(cfg, w, b)
    read = lambda n, rows: torch.from_numpy(np.fromfile(os.path.join(out, f"{n}.f32"), dtype="<f4").reshape(rows, vocab).copy())
    assert _rel_rms(read(0, 2), wa[[0, 32]]) < FLOAT_LOGITS
    assert _rel_rms(read(1, 1), wb[[19]]) < FLOAT_LOGITS
    assert _rel_rms(read(2, 1), wa[[68]]) < FLOAT_LOGITS and _rel_rms(read(3, 1), wa[[69]]) < FLOAT_LOGITS
