"""Nosedra on the GPU against the plain implementation (tests/plain_nosedra.py): every mechanism
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

import plain_nosedra as P
from tiny_nosedra import CONFIGS, SEEDS, STD_BY_SUFFIX, config

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


# Float arithmetic against the plain model in double.  A recurrence's exponents have arguments of the size of the gates'
# cap (tens), known to 2^-24 of that, and the normaliser n . q cancels; a rotation's angle at position p is known to
# p * 2^-24; a state that has moved T times has drifted T roundings, all one way where the decay is almost 1.  Whatever
# the design adds shows at 5e-3 and more when left out (test_what_the_design_adds_would_show_if_left_out).
FLOAT_WALK = 1e-4             # a row of a recurrence's output, and its state, over tens of tokens
FLOAT_LONG_WALK = 5e-4        # the same after 600 tokens
FLOAT_ROTATION = 1e-4         # rotated and normed rows at positions beyond a thousand
FLOAT_LOGITS = 3e-4           # a row of logits, a layer's stream
FLOAT_SAME = 3e-5             # the same logits by another cut or in another batch


def _within_noise(err: torch.Tensor, noise: torch.Tensor, what: str) -> None:
    """`err`: per row, the engine's bfloat16 error; `noise`: per row, how far the plain model moves
    when it rounds to bfloat16 every tensor that a 16-bit engine may keep in 16 bits, and nothing of
    what the design computes in 32 bits.  A row's limit is three times its noise (at least three
    times the median row's: one draw of the noise can be small by chance).  At most three rows in a
    hundred (or one) may exceed it, none two and a half times it.  A wrong key, sink, state or tail
    puts the rows it touches at order one, tens of times the usual row's noise; the float32 runs of
    the same tests are the sharp ones."""
    limit = 3.0 * torch.maximum(noise, noise.median())
    over, far = int((err > limit).sum()), int((err > 2.5 * limit).sum())
    worst = int((err / limit).argmax())
    assert over <= max(1, 0.03 * err.numel()) and far == 0, \
        f"{what}: {over} of {err.numel()} rows over their limit, {far} far over; row {worst}: {float(err[worst]):.2e} (limit {float(limit[worst]):.2e})"


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


# five steps of three requests: one token, a few, many; a request left out of a step; pairs and singles at the end
PLAN = [[("a", 1), ("b", 40)], [("b", 1), ("c", 7), ("a", 2)], [("a", 9), ("c", 1)], [("c", 1), ("a", 2), ("b", 1)], [("b", 1)]]
TOTAL = {"a": 14, "b": 43, "c": 9}
SLOT_OF = {"a": 3, "b": 0, "c": 1}


def _walk_plan(rows_of, gates_of, call):
    """Runs `call(rows, gates, ctx)` over PLAN, returns each request's outputs in order."""
    got = {r: [] for r in TOTAL}
    at = {r: 0 for r in TOTAL}
    for step in PLAN:
        ctx = _Step([n for _, n in step], [at[r] for r, _ in step], [SLOT_OF[r] for r, _ in step])
        rows = torch.cat([rows_of[r][at[r]:at[r] + n] for r, n in step]).to(DEV)
        gates = torch.cat([gates_of[r][at[r]:at[r] + n] for r, n in step]).to(DEV)
        o = call(rows, gates, ctx)
        i = 0
        for r, n in step:
            got[r].append(o[i:i + n].cpu())
            i += n
            at[r] += n
    return {r: torch.cat(v) for r, v in got.items()}


# ---------------------------------------------------------------------------
# the mechanisms alone
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, dk, dv, cap", [(2, 10, 24, 6.0), (5, 32, 40, 12.0), (1, 136, 20, 4.0), (3, 72, 50, 1.0), (2, 256, 16, 30.0),
                                            (4, 64, 33, 8.0)])
def test_the_matrix_memory_walks_every_entry_from_its_slots_state(dtype, H, dk, dv, cap):
    """Exponential gates with their cap, the running maximum from 0, the normaliser and the floor of
    the denominator, against the plain recurrence over whole sequences; states in slots 3, 0 and 1 of
    five.  The gates' pre-activations are spread wide, so that the cap bends them and the maximum
    moves both ways."""
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(dk + dv)
    qk, vv = H * dk, H * dv
    pad = 3 if dk % 16 else 8
    proj = {r: torch.randn(n, pad + 2 * qk + vv + 5, generator=g).to(DT[dtype]) for r, n in TOTAL.items()}
    z = {r: torch.randn(n, 2 * H, generator=g) * 1.5 * cap for r, n in TOTAL.items()}
    b_i, b_f = torch.randn(H, generator=g), torch.randn(H, generator=g) + 2.0
    state = torch.zeros(5, *ops.walk_state_shape(H, dk, dv, ops.WALK_EXP_GATES), device=DEV)
    state[2].fill_(9.0)                                          # a slot no entry names
    scale = dk ** -0.5

    def call(rows, gates, ctx):
        return ops.state_walk(rows, pad, pad + qk, pad + 2 * qk, 1, gates, (b_i.to(DEV), b_f.to(DEV)), cap, scale,
                              ops.WALK_EXP_GATES, state, ctx, H, dk, dv)

    got = _walk_plan(proj, z, call)
    for r, n in TOTAL.items():
        p, zz = proj[r].double(), z[r].double()
        log_i = P.capped(zz[:, :H] + b_i.double(), cap)
        log_f = P.log_sigmoid(P.capped(zz[:, H:] + b_f.double(), cap))
        q, k = p[:, pad:pad + qk].reshape(n, H, dk) * scale, p[:, pad + qk:pad + 2 * qk].reshape(n, H, dk)
        v = p[:, pad + 2 * qk:pad + 2 * qk + vv].reshape(n, H, dv)
        want = P.matrix_memory(q, k, v, log_i, log_f)
        assert got[r].dtype == torch.float32
        assert _rel_rms(got[r], want.reshape(n, -1)) < FLOAT_WALK, r        # float arithmetic in both dtypes
        # what the slot holds in the end: S, n and m of the plain recurrence
        S, nn, m = torch.zeros(H, dk, dv, dtype=torch.float64), torch.zeros(H, dk, dtype=torch.float64), torch.zeros(H, dtype=torch.float64)
        for t in range(n):
            m_new = torch.maximum(log_f[t] + m, log_i[t])
            keep, take = torch.exp(log_f[t] + m - m_new), torch.exp(log_i[t] - m_new)
            S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
            nn = keep[:, None] * nn + take[:, None] * k[t]
            m = m_new
        gS, gn, gm = ops.walk_state_matrices(state[SLOT_OF[r]], dk, dv, ops.WALK_EXP_GATES)
        assert _rel_rms(gS.reshape(1, -1), S.reshape(1, -1)) < FLOAT_WALK, f"S of {r}"
        assert _rel_rms(gn.reshape(1, -1), nn.reshape(1, -1)) < FLOAT_WALK, f"n of {r}"
        assert float((gm.double().cpu() - m).abs().max()) < 1e-4, f"m of {r}"
    assert float((state[2] - 9.0).abs().max()) == 0.0 and float(state[4].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_matrix_memorys_first_tokens_and_its_denominators_floor(dtype):
    """The maximum starts at 0, not far below: a first token whose input gate lies far below 0 enters
    with the weight exp(i) and not 1 (the denominator is exp(-m), about 1); a query orthogonal to
    every key so far gives exactly nothing."""
    from sharpinference_amd import ops

    H, dk, dv, cap = 1, 32, 8, 20.0
    T = 6
    k = torch.zeros(T, dk)
    q = torch.zeros(T, dk)
    k[:, 0] = 1.0
    q[:, 0] = 1.0
    q[4] = 0.0
    q[4, 1] = 1.0                                                # orthogonal to every key so far: n . q = 0
    v = torch.arange(1, T * dv + 1, dtype=torch.float32).reshape(T, dv) / 8
    proj = torch.cat([q, k, v], dim=1).to(DT[dtype])
    z = torch.tensor([[-9.0, 3.0], [-2.0, 3.0], [1.0, -1.0], [4.0, 0.0], [0.0, 2.0], [0.5, 2.0]])
    zero = torch.zeros(H, device=DEV)
    state = torch.zeros(1, *ops.walk_state_shape(H, dk, dv, ops.WALK_EXP_GATES), device=DEV)
    ctx = _Step([T], [0], [0])
    o = ops.state_walk(proj.to(DEV), 0, dk, 2 * dk, 1, z.to(DEV), (zero, zero), cap, 1.0, ops.WALK_EXP_GATES, state, ctx, H, dk, dv)
    p = proj.double()
    log_i, log_f = P.capped(z[:, :1].double(), cap), P.log_sigmoid(P.capped(z[:, 1:].double(), cap))
    want = P.matrix_memory(p[:, :dk].reshape(T, 1, dk), p[:, dk:2 * dk].reshape(T, 1, dk), p[:, 2 * dk:].reshape(T, 1, dv), log_i, log_f)
    assert _rel_rms(o, want.reshape(T, -1)) < FLOAT_WALK
    # token 0: m_1 = max(f_0 + 0, i_0) = f_0, the value enters with exp(i_0 - m_1), the denominator is exp(-m_1) (+ the floor)
    i0, m1 = float(log_i[0]), float(log_f[0])
    assert i0 < -8 and -0.1 < m1 < 0
    assert _rel_rms(o[:1], math.exp(i0 - m1) / (math.exp(-m1) + 1e-6) * p[:1, 2 * dk:]) < 1e-5
    assert float(o[4].abs().max()) == 0.0                        # S^T q = 0 for the orthogonal query, whatever the denominator


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, G, N, dv", [(3, 1, 10, 8), (6, 2, 40, 24), (8, 2, 64, 16), (2, 1, 72, 50), (3, 3, 136, 12), (4, 4, 20, 6),
                                         (2, 2, 256, 9)])
def test_the_state_space_walks_every_entry_from_its_slots_state(dtype, H, G, N, dv):
    """Step sizes through their softplus (no clamp: some far below 0, some large), decays
    exp(-exp(A_log) dt), B and C shared by the heads of a group, the skip D x."""
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(N + dv + H)
    inner = H * dv
    C = inner + 2 * G * N
    xbc = {r: torch.randn(n, C, generator=g).to(DT[dtype]) for r, n in TOTAL.items()}
    z = {r: torch.randn(n, H + 2, generator=g) * 3.0 for r, n in TOTAL.items()}      # (two columns more than the heads: a wider row)
    dt_bias, a_log, d_skip = torch.randn(H, generator=g), torch.randn(H, generator=g) * 0.7, torch.randn(H, generator=g)
    state = torch.zeros(5, *ops.walk_state_shape(H, N, dv, ops.WALK_STATE_SPACE), device=DEV)
    state[4].fill_(-3.0)

    def call(rows, gates, ctx):
        return ops.state_walk(rows, inner + G * N, inner, 0, H // G, gates, (dt_bias.to(DEV), a_log.to(DEV), d_skip.to(DEV)),
                              0.0, 1.0, ops.WALK_STATE_SPACE, state, ctx, H, N, dv)

    got = _walk_plan(xbc, z, call)
    for r, n in TOTAL.items():
        u = xbc[r].double()
        dt = P.softplus(z[r][:, :H].double() + dt_bias.double())
        x, B, Cc = u[:, :inner].reshape(n, H, dv), u[:, inner:inner + G * N].reshape(n, G, N), u[:, inner + G * N:].reshape(n, G, N)
        want = P.state_space_scan(x, B, Cc, dt, a_log.double(), d_skip.double())
        assert _rel_rms(got[r], want.reshape(n, -1)) < FLOAT_WALK, r
        S = torch.zeros(H, N, dv, dtype=torch.float64)
        rep = H // G
        for t in range(n):
            decay = torch.exp(-torch.exp(a_log.double()) * dt[t])
            S = decay[:, None, None] * S + dt[t][:, None, None] * B[t].repeat_interleave(rep, 0)[:, :, None] * x[t][:, None, :]
        gS, _, _ = ops.walk_state_matrices(state[SLOT_OF[r]], N, dv, ops.WALK_STATE_SPACE)
        assert _rel_rms(gS.reshape(1, -1), S.reshape(1, -1)) < FLOAT_WALK, f"state of {r}"
    assert float((state[4] + 3.0).abs().max()) == 0.0 and float(state[2].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["gates", "space"])
def test_one_token_far_back_is_still_in_the_state(dtype, mode):
    """600 tokens whose forget gates (decays) are almost 1 and whose input weights are tiny but for the
    third token: the last query, aimed at that token's key, returns its value."""
    from sharpinference_amd import ops

    H, dk, dv, T, mark = 2, 32, 16, 600, 2
    g = torch.Generator().manual_seed(5)
    k = torch.randn(T, H, dk, generator=g) * 0.1
    q = torch.randn(T, H, dk, generator=g) * 0.1
    v = torch.randn(T, H, dv, generator=g)
    k[mark] = torch.nn.functional.normalize(torch.randn(H, dk, generator=g), dim=-1) * 4.0
    q[T - 1] = k[mark] / 4.0
    state_mode = ops.WALK_EXP_GATES if mode == "gates" else ops.WALK_STATE_SPACE
    state = torch.zeros(1, *ops.walk_state_shape(H, dk, dv, state_mode), device=DEV)
    ctx_of = lambda a, b: _Step([b - a], [a], [0])
    cuts = [0, 1, 3, 130, 131, 599, 600]                         # the marked token closes a portion of two
    outs = []
    if mode == "gates":
        z = torch.cat([torch.full((T, H), -8.0), torch.full((T, H), 12.0)], dim=1)
        z[mark, :H] = 2.0
        proj = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], dim=1).to(DT[dtype])
        zero = torch.zeros(H, device=DEV)
        for a, b in zip(cuts, cuts[1:]):
            outs.append(ops.state_walk(proj[a:b].to(DEV), 0, H * dk, 2 * H * dk, 1, z[a:b].to(DEV), (zero, zero), 14.0, 1.0,
                                       state_mode, state, ctx_of(a, b), H, dk, dv).cpu())
        p = proj.double()
        want = P.matrix_memory(p[:, :H * dk].reshape(T, H, dk), p[:, H * dk:2 * H * dk].reshape(T, H, dk), p[:, 2 * H * dk:].reshape(T, H, dv),
                               P.capped(z[:, :H].double(), 14.0), P.log_sigmoid(P.capped(z[:, H:].double(), 14.0)))
    else:
        z = torch.full((T, H), -9.0)                              # dt = softplus(-9): tiny steps, decays almost 1
        z[mark] = 1.0
        proj = torch.cat([v.reshape(T, -1), k.reshape(T, -1), q.reshape(T, -1)], dim=1).to(DT[dtype])
        par = (torch.zeros(H, device=DEV), torch.full((H,), -3.0, device=DEV), torch.zeros(H, device=DEV))
        for a, b in zip(cuts, cuts[1:]):
            outs.append(ops.state_walk(proj[a:b].to(DEV), H * dv + H * dk, H * dv, 0, 1, z[a:b].to(DEV), par, 0.0, 1.0,
                                       state_mode, state, ctx_of(a, b), H, dk, dv).cpu())
        p = proj.double()
        want = P.state_space_scan(p[:, :H * dv].reshape(T, H, dv), p[:, H * dv:H * dv + H * dk].reshape(T, H, dk),
                                  p[:, H * dv + H * dk:].reshape(T, H, dk), P.softplus(z.double()), torch.full((H,), -3.0).double(),
                                  torch.zeros(H).double())
    got = torch.cat(outs)
    assert _rel_rms(got, want.reshape(T, -1)) < FLOAT_LONG_WALK
    last, value = want[T - 1].reshape(1, -1), p[mark, (2 * H * dk if mode == "gates" else 0):][:H * dv].reshape(1, -1)
    cos = float((last * value).sum() / (last.norm() * value.norm()))
    assert cos > 0.98, cos                                       # the far token carries the last output


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode, H, G, dk, dv", [("gates", 2, 2, 32, 16), ("gates", 3, 3, 72, 20), ("gates", 1, 1, 136, 9),
                                               ("space", 4, 2, 40, 16), ("space", 2, 1, 128, 24), ("space", 3, 3, 10, 8)])
def test_long_entries_walked_in_segments_side_by_side(dtype, mode, H, G, dk, dv):
    """Three entries of 700, 5 and 257 tokens in one step, from states that earlier tokens left: cut into
    segments (each walked from nothing, the start states made one from the other, then walked again)
    against the plain recurrence over the whole sequences, and the states left in the slots against a
    walk of whole entries."""
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(dk * dv)
    before, lens, slots = [3, 40, 0], [700, 5, 257], [2, 0, 3]
    state_mode = ops.WALK_EXP_GATES if mode == "gates" else ops.WALK_STATE_SPACE
    cap = 6.0
    n_gate = 2 * H if mode == "gates" else H
    rows, zs = [], []
    for b, n in zip(before, lens):
        T = b + n
        q, k, v = torch.randn(T, G * dk, generator=g) * 0.5, torch.randn(T, G * dk, generator=g) * 0.5, torch.randn(T, H * dv, generator=g)
        rows.append((torch.cat([v, k, q], dim=1) if mode == "space" else torch.cat([q, k, v], dim=1)).to(DT[dtype]))
        z = torch.randn(T, n_gate, generator=g) * 2.0
        if mode == "gates":
            z[:, H:] += 3.0                                       # forget gates mostly open: the far past still counts
        else:
            z -= 3.0                                              # small steps: slow decays
        zs.append(z)
    if mode == "gates":
        par = (torch.randn(H, generator=g), torch.randn(H, generator=g))
        offs, rep, scale = (0, G * dk, 2 * G * dk), 1, dk ** -0.5
    else:
        par = (torch.randn(H, generator=g) * 0.5, torch.randn(H, generator=g) * 0.5 - 1.0, torch.randn(H, generator=g))
        offs, rep, scale = (H * dv + G * dk, H * dv, 0), H // G, 1.0
    dpar = tuple(p.to(DEV) for p in par)

    def run(segmented):
        state = torch.zeros(4, *ops.walk_state_shape(H, dk, dv, state_mode), device=DEV)
        outs = []
        for part in (0, 1):                                       # what came before, then the long step
            ns = [b if part == 0 else n for b, n in zip(before, lens)]
            at = [0 if part == 0 else b for b in before]
            live = [i for i, n in enumerate(ns) if n > 0]
            ctx = _Step([ns[i] for i in live], [at[i] for i in live], [slots[i] for i in live])
            x = torch.cat([rows[i][at[i]:at[i] + ns[i]] for i in live]).to(DEV)
            z = torch.cat([zs[i][at[i]:at[i] + ns[i]] for i in live]).to(DEV)
            segments = None
            if segmented and part == 1:
                segs, ents = ops.gla_segments(ctx_lens := [ns[i] for i in live], ctx.cu_tokens.cpu().numpy())
                assert segs.shape[0] == sum((n + 127) // 128 for n in ctx_lens)
                segments = (torch.from_numpy(segs).to(DEV), torch.from_numpy(ents).to(DEV))
            o = ops.state_walk(x, offs[0], offs[1], offs[2], rep, z, dpar, cap, scale, state_mode, state, ctx, H, dk, dv,
                               segments=segments)
            outs.append((live, [ns[i] for i in live], o.cpu()))
        return outs[1], state

    (live, ns, seg_out), seg_state = run(True)
    (_, _, whole_out), whole_state = run(False)
    o = 0
    for i, n in zip(live, ns):
        p, z = rows[i].double(), zs[i].double()
        T = p.shape[0]
        if mode == "gates":
            log_i = P.capped(z[:, :H] + par[0].double(), cap)
            log_f = P.log_sigmoid(P.capped(z[:, H:] + par[1].double(), cap))
            want = P.matrix_memory(p[:, :H * dk].reshape(T, H, dk) * scale, p[:, H * dk:2 * H * dk].reshape(T, H, dk),
                                   p[:, 2 * H * dk:].reshape(T, H, dv), log_i, log_f)
        else:
            want = P.state_space_scan(p[:, :H * dv].reshape(T, H, dv), p[:, H * dv:H * dv + G * dk].reshape(T, G, dk),
                                      p[:, H * dv + G * dk:].reshape(T, G, dk), P.softplus(z + par[0].double()), par[1].double(),
                                      par[2].double())
        want = want.reshape(T, -1)[before[i]:]
        assert _rel_rms(seg_out[o:o + n], want) < FLOAT_LONG_WALK, f"entry {i}"
        assert _rel_rms(whole_out[o:o + n], want) < FLOAT_LONG_WALK, f"entry {i} whole"
        o += n
    for slot in slots:
        for a, b in zip(ops.walk_state_matrices(seg_state[slot], dk, dv, state_mode), ops.walk_state_matrices(whole_state[slot], dk, dv, state_mode)):
            if a is not None:
                scale_of = float(b.abs().max()) + 1e-30
                assert float((a - b).abs().max()) / scale_of < FLOAT_WALK, f"slot {slot}"
    assert float(seg_state[1].abs().max()) == 0.0                 # the slot no entry names


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("channels, taps, bias", [(29, 2, True), (64, 3, True), (200, 4, True), (24, 8, True), (40, 1, True), (16, 4, False)])
def test_the_biased_convolution_carries_its_tail_from_step_to_step(dtype, channels, taps, bias):
    """Three requests over five steps, portions shorter than the convolution's reach among them:
    silu(b + conv) against the plain convolution over whole sequences; the tails in slots 3, 0, 1."""
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(channels + taps)
    off, tailpad = 7, 4
    proj = {r: (torch.randn(n, off + channels + tailpad, generator=g) * 2).to(DT[dtype]) for r, n in TOTAL.items()}
    w = torch.randn(channels, taps, generator=g)
    b = torch.randn(channels, generator=g) if bias else None
    tail = torch.zeros(5, taps - 1, channels, device=DEV) if taps > 1 else None
    if tail is not None:
        tail[2].fill_(7.0)
    none = {r: torch.zeros(n, 1) for r, n in TOTAL.items()}

    def call(rows, _, ctx):
        return ops.short_conv(rows, off, channels, w.to(DEV), b.to(DEV) if bias else None, tail, ctx)

    got = _walk_plan(proj, none, call)
    for r, n in TOTAL.items():
        u = proj[r].double()[:, off:off + channels]
        want = P.silu(P.biased_convolution(u, w.double(), b.double() if bias else torch.zeros(channels).double()))
        assert got[r].dtype == DT[dtype]
        assert _rel_rms(got[r], want) < (2e-6 if dtype == "float32" else 6e-3), r
        if tail is not None:                                     # the slot holds the request's last taps - 1 inputs
            keep = min(taps - 1, n)
            assert float((tail[SLOT_OF[r]][-keep:].cpu().double() - u[-keep:]).abs().max()) == 0.0
    if tail is not None:
        assert float((tail[2] - 7.0).abs().max()) == 0.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T, groups, size, act, first", [(1, 5, 40, "sigmoid", False), (19, 2, 64, "silu", True), (70, 3, 8, "silu", True),
                                                         (9, 1, 100, "silu", True), (33, 2, 50, "sigmoid", False), (5, 4, 6, "silu", False)])
def test_parts_normed_each_by_its_own_rms_with_a_gate_before_or_after(dtype, T, groups, size, act, first):
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(T + size)
    N, off = groups * size, 11
    o = torch.randn(T, N, generator=g) * torch.rand(T, 1, generator=g) * 5
    w = torch.randn(N, generator=g)
    gp = (torch.randn(T, off + N + 3, generator=g) * 2).to(DT[dtype])
    eps = 1e-3
    out = ops.group_norm_gate(o.to(DEV), w.to(DEV), eps, groups, DT[dtype], gp.to(DEV), off,
                              ops.GATE_SILU if act == "silu" else ops.GATE_SIGMOID_ACT, gate_first=first)
    z = gp.double()[:, off:off + N]
    gate = P.silu(z) if act == "silu" else torch.sigmoid(z)
    od = o.double()
    if first:
        want = P.unit_rms((od * gate).view(T, groups, size), eps).reshape(T, N) * w.double()
    else:
        want = P.unit_rms(od.view(T, groups, size), eps).reshape(T, N) * w.double() * gate
    assert out.dtype == DT[dtype]
    assert _rel_rms(out, want) < (2e-6 if dtype == "float32" else 5e-3)
    if groups > 1:                                               # one norm over the whole row would be something else
        other = P.unit_rms(od * gate if first else od, eps) * w.double() * (1.0 if first else gate)
        assert _rel_rms(other, want) > 0.02


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T, N", [(1, 72), (9, 256), (70, 1000)])
def test_a_scaled_sum_of_branches_joins_the_stream_in_float(dtype, T, N):
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(T + N)
    h = torch.randn(T, N, generator=g) * 3
    a, b = torch.randn(T, N, generator=g).to(DT[dtype]), torch.randn(T, N, generator=g).to(DT[dtype])
    hd = h.clone().to(DEV)
    out = ops.stream_add(hd, ops.BranchSum([a.to(DEV), b.to(DEV)], (1.3, -0.7)), DT[dtype])
    want = h.double() + 1.3 * a.double() + -0.7 * b.double()
    assert _rel_rms(hd, want) < 2e-6                             # the stream itself stays float
    assert out.dtype == DT[dtype] and _rel_rms(out, want) < (2e-6 if dtype == "float32" else 5e-3)
    alone = ops.BranchSum([a.to(DEV), b.to(DEV)], (0.5, 2.0)).tensor()
    assert alone.dtype == torch.float32 and _rel_rms(alone, 0.5 * a.double() + 2.0 * b.double()) < 2e-6
    h2 = h.clone().to(DEV)
    assert ops.stream_add(h2, None) is None and float((h2.cpu() - h).abs().max()) == 0.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_token_input_the_biased_feed_forward_and_the_output_gate(dtype):
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(12)
    T, D, V, L = 21, 5, 37, 4
    gate = (torch.randn(T, D, generator=g) * 2).to(DT[dtype])
    table = torch.randn(V, L * D, generator=g).to(DT[dtype])
    ids = torch.randint(0, V, (T,), generator=g, dtype=torch.int32)
    tol = 2e-6 if dtype == "float32" else 6e-3
    for layer in (0, 2, 3):
        out = ops.side_gate(gate.to(DEV), ids.to(DEV), table.to(DEV), layer * D)
        want = P.gelu_tanh(gate.double()) * table.double()[ids.long()][:, layer * D:(layer + 1) * D]
        assert _rel_rms(out, want) < tol, layer
    # h += unit_rms(y) * w with a plain weight
    h, y, w = torch.randn(T, 72, generator=g), (torch.randn(T, 72, generator=g) * 4).to(DT[dtype]), torch.randn(72, generator=g)
    hd = h.clone().to(DEV)
    ops.norm_add(hd, y.to(DEV), w.to(DEV), 1e-5)
    assert _rel_rms(hd, h.double() + P.unit_rms(y.double(), 1e-5) * w.double()) < 2e-6
    # gelu_tanh(gate + b) * (up + b)
    I = 40
    gu, bias = (torch.randn(T, 2 * I, generator=g) * 2).to(DT[dtype]), torch.randn(2 * I, generator=g)
    act = ops.gated_act(gu.to(DEV), None, ops.ACT_GELU_TANH, bias=bias.to(DEV))
    z = gu.double() + bias.double()
    assert _rel_rms(act, P.gelu_tanh(z[:, :I]) * z[:, I:]) < tol
    assert _rel_rms(P.silu(z[:, :I]) * z[:, I:], P.gelu_tanh(z[:, :I]) * z[:, I:]) > 0.02       # (the other activation is elsewhere)
    # o * sigmoid(gate columns of a wider row)
    o, wide = torch.randn(T, 24, generator=g).to(DT[dtype]), (torch.randn(T, 50, generator=g) * 2).to(DT[dtype])
    got = ops.sigmoid_gate(o.to(DEV), wide.to(DEV), 26)
    assert _rel_rms(got, o.double() * torch.sigmoid(wide.double()[:, 26:])) < tol


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, G, d, e, dims, factor", [(4, 2, 12, 20, 4, 4.0), (6, 1, 8, 6, 8, 1.0), (8, 2, 128, 128, 32, 4.0), (4, 2, 64, 64, 64, 8.0),
                                                      (2, 1, 24, 40, 24, 1.5), (4, 4, 16, 16, 0, 1.0), (8, 2, 32, 32, 16, 2.0)])
def test_split_half_rotation_then_unit_norm_and_the_cache_write(dtype, H, G, d, e, dims, factor):
    """Two requests in two steps each on shuffled pages: rotated (leading `dims` elements, halves
    paired, frequencies divided by the factor) and then normed q, and the cached keys and values,
    against the plain pieces; the gate's columns behind q, k and v are left alone."""
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(H * 100 + d)
    ps, eps = 16, 1e-5
    qn, kn, vn, extra = H * d, G * d, G * e, H * e
    lens = {"a": [19, 1], "b": [2, 30]}
    total = {r: sum(v) for r, v in lens.items()}
    base = {"a": 0, "b": 1000}                                  # (b's positions begin far out: large angles in float)
    rows = {r: (torch.randn(total[r], qn + kn + vn + extra, generator=g) * 2).to(DT[dtype]) for r in lens}
    rot = {"base": 5000.0, "dims": dims, "scaling": {"factor": factor}}
    freqs = P.frequencies(rot) if dims else []
    if dims:
        assert abs(freqs[-1] - 5000.0 ** (-(dims - 2) / dims) / factor) < 1e-12
    pages = 8
    perm = torch.randperm(pages, generator=g).tolist()
    page_of = {"a": perm[:2], "b": perm[2:4]}
    kc = torch.zeros(pages, G, ps, d, dtype=DT[dtype], device=DEV)
    vc = torch.zeros(pages, G, e, ps, dtype=DT[dtype], device=DEV)
    inv_freq = torch.tensor(freqs, dtype=torch.float32, device=DEV) if dims else None
    got_q = {r: [] for r in lens}
    at = {r: 0 for r in lens}
    for step in range(2):
        entries = [(r, lens[r][step]) for r in lens]
        x = torch.cat([rows[r][at[r]:at[r] + n] for r, n in entries]).to(DEV)
        keep = x.clone()
        pos = torch.tensor([base[r] + at[r] + i for r, n in entries for i in range(n)], dtype=torch.int32, device=DEV)
        slots = torch.tensor([page_of[r][(at[r] + i) // ps] * ps + (at[r] + i) % ps for r, n in entries for i in range(n)],
                             dtype=torch.int32, device=DEV)
        q = ops.rope_kv(x, kc, vc, slots, pos, inv_freq, True, eps, None, H, G, d, ops.PAIRS_HALF_SPLIT, vd=e, extra_columns=extra)
        assert float((x[:, qn + kn + vn:] - keep[:, qn + kn + vn:]).abs().max()) == 0.0
        i = 0
        for r, n in entries:
            got_q[r].append(q[i:i + n].cpu())
            i += n
            at[r] += n
    tol = 3e-6 if dtype == "float32" else 6e-3
    for r in lens:
        u = rows[r].double()
        pos = base[r] + torch.arange(total[r])
        q, k, v = u[:, :qn].reshape(-1, H, d), u[:, qn:qn + kn].reshape(-1, G, d), u[:, qn + kn:qn + kn + vn].reshape(-1, G, e)
        if dims:
            q, k = P.rotate_halves(q, pos, freqs), P.rotate_halves(k, pos, freqs)
        q, k = P.unit_rms(q, eps), P.unit_rms(k, eps)
        assert _rel_rms(torch.cat(got_q[r]).reshape(total[r], -1), q.reshape(total[r], -1)) < (FLOAT_ROTATION if dtype == "float32" else tol), r
        gk = torch.stack([kc[page_of[r][p // ps], :, p % ps] for p in range(total[r])]).cpu()
        gv = torch.stack([vc[page_of[r][p // ps], :, :, p % ps] for p in range(total[r])]).cpu()
        assert _rel_rms(gk.reshape(total[r], -1), k.reshape(total[r], -1)) < (FLOAT_ROTATION if dtype == "float32" else tol), r
        assert _rel_rms(gv.reshape(total[r], -1), v.reshape(total[r], -1)) < 1e-7, r


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


def _attention_case(S, H, G, d, e, dtype, seed, marked=None, sharpen=30.0):
    """Random queries, keys and values; with `marked`, the last position's queries point at that key
    (and the key is made long), so that its score stands far out."""
    g = torch.Generator().manual_seed(seed)
    q, k, v = torch.randn(S, H, d, generator=g), torch.randn(S, G, d, generator=g), torch.randn(S, G, e, generator=g)
    if marked is not None:
        k[marked] *= 3.0
        for h in range(H):
            kk = k[marked, h // (H // G)]
            q[S - 1, h] = kk * (sharpen / kk.pow(2).sum()) + 0.05 * q[S - 1, h]
    return q.to(DT[dtype]), k.to(DT[dtype]), v.to(DT[dtype])


KERNELS = [("float32", "float", "all"), ("bfloat16", "float", "all"), ("bfloat16", "matrix cores", "tiles"),
           ("bfloat16", "matrix cores", "singles")]


def _attend(q, kc, vc, bt, positions, how, scale, H, G, d, e, sink):
    from sharpinference_amd import ops
    from sharpinference_amd.cache.spec import WINDOW_NONE

    S = int(positions.max()) + 1
    sink = sink.to(DEV) if isinstance(sink, torch.Tensor) else sink
    if how == "all":
        return ops.attention_generic(q, kc, vc, bt.to(DEV), torch.zeros(q.shape[0], dtype=torch.int32, device=DEV), positions.to(DEV),
                                     WINDOW_NONE, 0, scale, H, G, d, e, sink=sink)
    assert d == e and ops.decode_attention_ok(q.dtype, d) and ops.prefill_attention_ok(q.dtype, d)
    ctx = _Ctx(positions, tiles=how == "tiles", singles=how == "singles")
    return ops.attention(q, kc, vc, _Group(bt, S), ctx, WINDOW_NONE, 0, scale, H, G, d, e, sink=sink)


@pytest.mark.parametrize("dtype, kernel, how", KERNELS)
@pytest.mark.parametrize("S, H, G, d, e", [(70, 4, 2, 64, 64), (200, 8, 2, 128, 128), (131, 2, 1, 32, 32), (90, 6, 6, 64, 64), (50, 4, 2, 12, 20),
                                           (77, 6, 1, 8, 6)])
def test_attention_with_a_learned_sink_per_head(dtype, kernel, how, S, H, G, d, e):
    """Sinks from far below the scores (no effect) to far above (the head's output shrinks to
    almost nothing), a different one for every head."""
    if kernel == "matrix cores" and (d != e or d % 32):
        pytest.skip("the float kernel serves this size")
    q, k, v = _attention_case(S, H, G, d, e, dtype, seed=S)
    sink = torch.linspace(-6.0, 7.0, H)
    scale = 1.7 / math.sqrt(d)
    kc, vc, bt = _paged(k, v, dtype, seed=S)
    pos = torch.arange(S, dtype=torch.int32)
    out = _attend(q.reshape(S, -1).to(DEV), kc, vc, bt, pos, how, scale, H, G, d, e, sink)
    want = P.sink_attention(q.double(), k.double(), v.double(), scale, sink.double())
    assert _rel_rms(out.reshape(S, -1), want.reshape(S, -1)) < (3e-6 if dtype == "float32" else 1.5e-2)
    # neither a sink of score 0 for every head nor none at all is the same thing
    for other in (torch.zeros(H).double(), torch.full((H,), -60.0).double()):
        assert _rel_rms(P.sink_attention(q.double(), k.double(), v.double(), scale, other).reshape(S, -1), want.reshape(S, -1)) > 0.05
    # the first token sees itself and the sink only: v_0 * 1 / (1 + exp(sink - score))
    s0 = (q[0].double() * k[0].double().repeat_interleave(H // G, 0)).sum(-1) * scale
    first = v[0].double().repeat_interleave(H // G, 0) / (1.0 + torch.exp(sink.double() - s0))[:, None]
    assert _rel_rms(want[0].reshape(1, -1), first.reshape(1, -1)) < 1e-9


@pytest.mark.parametrize("dtype, kernel, how", KERNELS)
@pytest.mark.parametrize("S, marked", [(691, 0), (691, 1), (691, 15), (691, 16), (691, 255), (691, 256), (691, 640), (691, 689), (691, 690),
                                       (130, 127), (129, 128), (65, 0), (17, 0)])
def test_one_key_among_hundreds_is_found_behind_a_sink(dtype, kernel, how, S, marked):
    """The last position's queries point at one long key: far back, at a page's first and last place,
    at a tile's edge, the first key of all and the token's own.  With a sink above every other score
    but the marked one's, the result is that key's value; a lost key would leave the sink alone and
    a result near zero."""
    H, G, d = 4, 2, 64
    q, k, v = _attention_case(S, H, G, d, d, dtype, seed=S + marked, marked=marked)
    sink = torch.full((H,), 12.0)                                # (the marked key scores 30, the others within +-8)
    kc, vc, bt = _paged(k, v, dtype, seed=marked)
    if how == "tiles":
        rows, pos = q.reshape(S, -1), torch.arange(S, dtype=torch.int32)
    else:
        rows, pos = q[S - 1:].reshape(1, -1), torch.tensor([S - 1], dtype=torch.int32)
    out = _attend(rows.to(DEV), kc, vc, bt, pos, how, 1.0, H, G, d, d, sink)[-1:].cpu()
    want = P.sink_attention(q.double(), k.double(), v.double(), 1.0, sink.double())[S - 1].reshape(1, -1)
    value = torch.stack([v[marked, h // (H // G)] for h in range(H)]).double().reshape(1, -1)
    assert _rel_rms(want, value) < 0.05                          # the marked key carries the result
    assert _rel_rms(out, want) < (3e-6 if dtype == "float32" else 1.5e-2)


# ---------------------------------------------------------------------------
# the engine
# ---------------------------------------------------------------------------
@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    from sharpinference_amd import load_config
    from sharpinference_amd.weights.loader import write_random_model

    out = {}
    for name in CONFIGS:
        d = str(tmp_path_factory.mktemp("nosedra_" + name))
        write_random_model(load_config(config(name)), d, SEEDS[name], std=0.1, std_by_suffix=STD_BY_SUFFIX)
        out[name] = d
    return out


@functools.lru_cache(maxsize=4)
def _plain_model(d):
    return P.read_config(d), P.load_weights(d, torch.float64)


def _engine(d, dtype, **kw):
    from sharpinference_amd.engine import Engine

    args = dict(dtype=dtype, device=DEV, max_num_seqs=4, kv_tokens=1024, max_model_len=1024)
    args.update(kw)
    return Engine(d, **args)


def _run(eng, reqs, steps, free=True):
    """steps: lists of (request id, number of its next tokens).  Returns per request the logits at
    every position."""
    from sharpinference_amd.engine import StepEntry

    at = {r: 0 for r in reqs}
    logits = {r: [] for r in reqs}
    for step in steps:
        entries = []
        for r, n in step:
            if at[r] == 0:
                eng.add_request(r)
            entries.append(StepEntry(r, reqs[r][at[r]:at[r] + n], list(range(n))))
        out = eng.step(entries).cpu()
        o = 0
        for r, n in step:
            logits[r].append(out[o:o + n])
            o += n
            at[r] += n
            if at[r] == len(reqs[r]) and free:
                eng.free_request(r)
    return {r: torch.cat(v) for r, v in logits.items()}


@functools.lru_cache(maxsize=64)
def _plain_logits(d, toks, rounded=False):
    cfg, w = _plain_model(d)
    return P.forward(cfg, w, list(toks), store=P.store_bf16 if rounded else P._same)


def _check(d, dtype, reqs, got, what):
    for r, toks in reqs.items():
        want = _plain_logits(d, tuple(toks))
        err = _rel_rows(got[r], want)
        if dtype == "float32":
            assert float(err.max()) < FLOAT_LOGITS, f"{what}, request {r}: {float(err.max()):.2e} at row {int(err.argmax())}"
        else:
            _within_noise(err, _rel_rows(_plain_logits(d, tuple(toks), True), want), f"{what}, request {r}")


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
@pytest.mark.parametrize("name", ["odd", "even", "wide"])
def test_every_layers_stream_agrees_with_the_plain_model(model_dirs, name, dtype):
    """The residual sum after every layer of a 40-token prompt, in float as the engine keeps it."""
    from sharpinference_amd.engine import StepEntry

    d = model_dirs[name]
    cfg, w = _plain_model(d)
    toks = _tokens(40, CONFIGS[name]["vocab"], 9)
    eng = _engine(d, dtype)
    caught = []
    for b in eng.model.blocks:
        def fwd(stream, ctx, cache, orig=b.forward):
            orig(stream, ctx, cache)
            assert stream.h.dtype == torch.float32 and stream.pending_norm is None
            rest = stream.pending_tensor()                       # (a layer without a token input leaves its last branch to the next norm)
            caught.append((stream.h if rest is None else stream.h + rest.float()).clone())
        b.forward = fwd
    eng.add_request("x")
    eng.step([StepEntry("x", toks, [39])])
    eng.free_request("x")
    want, rounded = [], []
    P.forward(cfg, w, toks, layers_out=want)
    P.forward(cfg, w, toks, layers_out=rounded, store=P.store_bf16)
    assert len(caught) == len(want)
    for i, (a, b, c) in enumerate(zip(caught, want, rounded)):
        if dtype == "float32":
            assert _rel_rms(a, b) < FLOAT_LOGITS, f"layer {i}: {_rel_rms(a, b):.2e}"
        else:
            _within_noise(_rel_rows(a, b), _rel_rows(c, b), f"layer {i}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["odd", "even", "wide"])
def test_whole_prompts_portions_and_decoding_agree_with_the_plain_model(model_dirs, name, dtype):
    d = model_dirs[name]
    vocab = CONFIGS[name]["vocab"]
    eng = _engine(d, dtype)
    toks = _tokens(150, vocab, 1)
    ways = {
        "whole": [150],
        "decoded one by one": [1] * 3 + [99] + [1] * 48,          # the first tokens alone, then a long tail through page borders
        "portions": _cuts(150, [2, 3, 17, 2, 64, 5, 16, 1, 31]),
        "pairs": [2] * 75,
    }
    first = None
    for what, cuts in ways.items():
        got = _run(eng, {what: toks}, [[(what, n)] for n in cuts])
        _check(d, dtype, {what: toks}, got, f"{name} {dtype} {what}")
        if dtype == "float32":
            first = got[what] if first is None else first
            assert _rel_rms(got[what], first) < FLOAT_SAME, f"{what}: the cut changes the logits"
    assert eng.runner.graph_replays > 0                           # decode steps ran from graphs, states and all
    eng.cache.check_invariants()
    assert not eng.cache.requests


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["odd", "wide"])
def test_a_long_prompt_agrees_with_its_portions(model_dirs, name, dtype):
    """700 tokens in one step and in portions of 100: the far keys of the attention and states that
    have moved hundreds of times."""
    d = model_dirs[name]
    toks = _tokens(700, CONFIGS[name]["vocab"], 8)
    eng = _engine(d, dtype, kv_tokens=2048)
    whole = _run(eng, {"w": toks}, [[("w", 700)]])
    _check(d, dtype, {"w": toks}, whole, f"{name} {dtype} 700 tokens at once")
    parts = _run(eng, {"p": toks}, [[("p", 100)] for _ in range(7)])
    _check(d, dtype, {"p": toks}, parts, f"{name} {dtype} 700 tokens in portions")
    if dtype == "float32":
        assert _rel_rms(whole["w"], parts["p"]) < FLOAT_SAME


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_first_tokens_and_a_long_decoded_tail(model_dirs, dtype):
    """Every token from the first decoded alone: 260 steps (the convolutions' tails start from zeros,
    the memories' maxima from 0), replayed from graphs."""
    d = model_dirs["odd"]
    toks = _tokens(260, CONFIGS["odd"]["vocab"], 7)
    eng = _engine(d, dtype)
    got = _run(eng, {"x": toks}, [[("x", 1)] for _ in toks])
    _check(d, dtype, {"x": toks}, got, f"decoded from the first token, {dtype}")
    assert eng.runner.graph_replays >= 250
    assert all(g.pool.num_free == g.pool.num_pages for g in eng.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["odd", "even"])
def test_unequal_requests_in_one_batch_give_what_each_gives_alone(model_dirs, name, dtype):
    d = model_dirs[name]
    vocab = CONFIGS[name]["vocab"]
    reqs = {"a": _tokens(90, vocab, 2), "b": _tokens(37, vocab, 3), "c": _tokens(130, vocab, 4), "d": _tokens(5, vocab, 5)}
    steps = [[("a", 29), ("b", 2)], [("a", 1), ("b", 33), ("c", 64)], [("c", 2), ("a", 1), ("d", 5), ("b", 1)],
             [("a", 59), ("c", 1), ("b", 1)], [("c", 63)]]
    eng = _engine(d, dtype)
    got = _run(eng, reqs, steps)
    _check(d, dtype, reqs, got, f"mixed {dtype}")
    if dtype == "float32":
        for r, toks in reqs.items():
            alone = _run(eng, {r: toks}, [[(r, len(toks))]])
            assert _rel_rms(got[r], alone[r]) < FLOAT_SAME, f"{r}: the batch changes the logits"
    eng.cache.check_invariants()


def test_pages_and_slots_are_given_back_and_used_again(model_dirs):
    """Two state slots and a pool of a dozen pages serve ten requests in turn: a matrix, a maximum or
    a tail that a request before left in its slot, or a key in a page used again, would show."""
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
        if what == "no sink":
            each(".sink", lambda t: torch.full_like(t, -60.0))
        elif what == "a sink of score 0":
            each(".sink", torch.zeros_like)
        elif what == "frequencies as they are":
            for l in c["layers"]:
                if l["type"] == "parallel" and l["mixer"]["left"].get("rot"):
                    l["mixer"]["left"]["rot"].pop("scaling", None)
        elif what == "no rotation":
            for l in c["layers"]:
                if l["type"] == "parallel":
                    l["mixer"]["left"].pop("rot", None)
        elif what == "the scales exchanged":
            for l in c["layers"]:
                if l["type"] == "parallel":
                    m = l["mixer"]
                    m["left_scale"], m["right_scale"] = m["right_scale"], m["left_scale"]
        elif what == "gates without a cap":
            for l in c["layers"]:
                if l["type"] == "parallel":
                    l["mixer"]["right"]["gate_cap"] = 1e6
        elif what == "no gate biases":
            each(".i.b", torch.zeros_like), each(".f.b", torch.zeros_like)
        elif what == "norm weights as stored":
            for k in w:
                if k.endswith("norm1") or k.endswith("norm2") or k == "final.norm":
                    ww[k] = w[k] - 1.0
        elif what == "no token input":
            each("side.norm", torch.zeros_like)
        elif what == "another layer's slice of the side table":
            ww["side.embed"] = torch.roll(w["side.embed"], c["token_side"]["dim"], dims=1)
        elif what == "logits without a cap":
            c.pop("logit_softcap")
        elif what == "a convolution of the current token alone":
            def ident(t):
                o = torch.zeros_like(t)
                o[:, -1] = 1.0
                return o
            each(".conv", ident)
        elif what == "no convolution bias":
            each(".conv.b", torch.zeros_like)
        elif what == "no step bias":
            each(".dt_bias", torch.zeros_like)
        elif what == "no skip":
            each(".D", torch.zeros_like)
        elif what == "one norm over the whole row":
            for l in c["layers"]:
                if l["type"] == "mamba2":
                    l["mixer"]["norm_groups"] = 1
        elif what == "no feed-forward biases":
            for k in w:
                if ".mlp." in k and k.endswith(".b"):
                    ww[k] = torch.zeros_like(w[k])
        return float(_rel_rows(got, P.forward(c, ww, toks)).max())

    for what in ("no sink", "a sink of score 0", "frequencies as they are", "no rotation", "the scales exchanged", "gates without a cap",
                 "no gate biases", "norm weights as stored", "no token input", "another layer's slice of the side table",
                 "logits without a cap", "a convolution of the current token alone", "no convolution bias", "no step bias", "no skip",
                 "one norm over the whole row", "no feed-forward biases"):
        assert changed(what) > 5e-3, what


@pytest.mark.parametrize("name", ["odd", "even", "wide"])
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
