"""Nosedra without a GPU: the configuration reader, the tensors the model asks for, the memory each
layer gets, the frequency tables, and the plain implementation's own consistency (what the GPU
tests lean on)."""
import math

import pytest
import torch

import plain_nosedra as P
from tiny_nosedra import CONFIGS, config

from sharpinference_amd import load_config
from sharpinference_amd.cache.spec import KVSpec, MixedSpec, StateSpec, kv_of, states_of
from sharpinference_amd.config.base import ConfigError
from sharpinference_amd.config.nosedra import NosedraConfig
from sharpinference_amd.parts.position import LinearScaling, Rotary
from sharpinference_amd.registry import build_model, registered_architectures


def test_the_design_is_registered_and_its_configuration_round_trips():
    assert "Nosedra" in registered_architectures()
    for name in CONFIGS:
        cfg = load_config(config(name))
        assert isinstance(cfg, NosedraConfig)
        assert cfg.to_dict() == config(name)
        assert load_config(cfg.to_dict()) == cfg


def test_what_the_file_leaves_out_is_off():
    d = config("wide")
    cfg = load_config(d)
    assert cfg.side_dim == 0 and cfg.logit_softcap == 0.0 and cfg.layers[0].left.rot is None
    assert cfg.layers[0].ff == 32 and cfg.layers[2].ff == 0
    odd = load_config(config("odd"))
    assert odd.layers[2].left.rot.factor == 1.0 and odd.layers[1].left.rot.factor == 4.0
    model = build_model(cfg)
    assert not any(n.startswith("side.") or ".side." in n for n in model.param_specs())
    d["layers"][3]["mixer"]["left"].pop("kv_heads")
    d["layers"][3]["mixer"]["left"].pop("vdim")
    d["layers"][3]["mixer"]["left"].pop("scale")
    left = load_config(d).layers[3].left
    assert (left.kv_heads, left.vdim) == (2, 24) and left.scale == pytest.approx(24 ** -0.5)


@pytest.mark.parametrize("path, value, what", [
    (("layers", 1, "mixer", "left", "window"), 7, "window"),
    (("layers", 1, "mixer", "left", "rot", "scaling", "low"), 2.0, "low"),
    (("layers", 1, "mixer", "right", "tau"), 2.0, "tau"),
    (("layers", 0, "mixer", "dt_min"), 0.1, "dt_min"),
    (("layers", 1, "mixer", "middle"), {}, "middle"),
    (("token_side", "scale"), 2.0, "scale"),
    (("norm", "kind"), "layer", "kind"),
    (("loop",), {"start": 0}, "loop"),
])
def test_a_key_the_reader_does_not_know_is_refused_by_name(path, value, what):
    d = config("odd")
    at = d
    for k in path[:-1]:
        at = at[k]
    at[path[-1]] = value
    with pytest.raises(ConfigError, match=what):
        load_config(d)


@pytest.mark.parametrize("change, what", [
    (lambda d: d["layers"][1]["mixer"]["left"].update(kv_heads=3), "kv_heads"),
    (lambda d: d["layers"][1]["mixer"]["left"].update(dim=11), "dim"),
    (lambda d: d["layers"][1]["mixer"]["left"]["rot"].update(dims=14), "dims"),
    (lambda d: d["layers"][1]["mixer"]["left"]["rot"]["scaling"].update(factor=0.0), "factor"),
    (lambda d: d["layers"][1]["mixer"]["right"].update(gate_cap=0.0), "gate_cap"),
    (lambda d: d["layers"][0]["mixer"].update(groups=2), "groups"),
    (lambda d: d["layers"][0]["mixer"].update(norm_groups=5), "norm_groups"),
    (lambda d: d["layers"][0]["mixer"].update(conv=0), "conv"),
    (lambda d: d["layers"][0].update(type="attention"), "attention"),
    (lambda d: d["layers"][0]["mlp"].update(kind="moe"), "kind"),
    (lambda d: d.update(vocab=0), "vocab"),
])
def test_sizes_that_contradict_each_other_are_refused(change, what):
    d = config("odd")
    change(d)
    with pytest.raises(ConfigError, match=what):
        load_config(d)


def test_the_tensors_the_model_asks_for():
    cfg = load_config(config("odd"))
    specs = {k: tuple(v.shape) for k, v in build_model(cfg).param_specs().items()}
    assert specs["embed"] == (101, 72) and specs["head"] == (101, 72) and specs["final.norm"] == (72,)
    assert specs["side.embed"] == (101, 4 * 5)
    # the state-space layer: z | x | B | C | dt rows of one matrix
    inner, G, N = 3 * 8, 1, 10
    assert specs["l0.mix.in"] == (2 * inner + 2 * G * N + 3, 72) and specs["l0.mix.conv"] == (inner + 2 * G * N, 2)
    assert specs["l0.mix.conv.b"] == (inner + 2 * G * N,) and specs["l0.mix.norm"] == (inner,) and specs["l0.mix.o"] == (72, inner)
    assert specs["l0.mix.A_log"] == specs["l0.mix.D"] == specs["l0.mix.dt_bias"] == (3,)
    # the parallel layer
    assert specs["l1.mix.left.q"] == (48, 72) and specs["l1.mix.left.k"] == (24, 72) and specs["l1.mix.left.v"] == (40, 72)
    assert specs["l1.mix.left.g"] == (80, 72) and specs["l1.mix.left.o"] == (72, 80) and specs["l1.mix.left.sink"] == (4,)
    assert specs["l1.mix.right.q"] == specs["l1.mix.right.k"] == (20, 72) and specs["l1.mix.right.v"] == specs["l1.mix.right.g"] == (48, 72)
    assert specs["l1.mix.right.i"] == specs["l1.mix.right.f"] == (2, 72) and specs["l1.mix.right.i.b"] == specs["l1.mix.right.f.b"] == (2,)
    assert specs["l1.mix.right.norm"] == (48,) and specs["l1.mix.right.o"] == (72, 48)
    assert specs["l1.mlp.gate"] == specs["l1.mlp.up"] == (56, 72) and specs["l1.mlp.down"] == (72, 56)
    assert specs["l1.mlp.gate.b"] == (56,) and specs["l1.mlp.down.b"] == (72,)
    assert "l2.mlp.gate" not in specs and "l2.norm2" not in specs and specs["l2.norm1"] == (72,)
    assert specs["l3.side.gate"] == (5, 72) and specs["l3.side.proj"] == (72, 5) and specs["l3.side.norm"] == (72,)
    # no tensor without a layer's prefix beyond these
    assert {k for k in specs if not k.startswith("l")} == {"embed", "head", "final.norm", "side.embed"}


def test_the_memory_each_layer_gets():
    from sharpinference_amd import ops

    model = build_model(load_config(config("odd")))
    specs = model.cache_specs()
    assert kv_of(specs[0]) is None and len(states_of(specs[0])) == 2          # the state and the convolution's tail
    assert states_of(specs[0])[1] == StateSpec((1, 3 * 8 + 2 * 10), torch.float32)
    assert states_of(specs[0])[0].shape == ops.walk_state_shape(3, 10, 8, ops.WALK_STATE_SPACE)
    assert kv_of(specs[1]) == KVSpec(2, 12, 0, 0, 20) and len(states_of(specs[1])) == 1
    assert states_of(specs[1])[0].shape == ops.walk_state_shape(2, 10, 24, ops.WALK_EXP_GATES)
    assert isinstance(specs[3], MixedSpec) and states_of(specs[3])[1].shape == (3, 4 * 6 + 2 * 4 * 20)
    wide = build_model(load_config(config("wide"))).cache_specs()
    assert isinstance(wide[1], StateSpec)                                     # one tap: no tail to carry
    assert model.decode_graph_safe()


def test_the_walks_state_layout_reads_back_as_matrices():
    from sharpinference_amd import ops

    for mode in (ops.WALK_EXP_GATES, ops.WALK_STATE_SPACE):
        for nh, dk, dv in ((2, 10, 24), (1, 136, 20), (3, 64, 8)):
            shape = ops.walk_state_shape(nh, dk, dv, mode)
            dkp = 32 if dk <= 32 else 64 if dk <= 64 else 128 if dk <= 128 else 256
            assert shape == (nh, (dv + 7) // 8, dkp * 8 + (dkp + 8 if mode == ops.WALK_EXP_GATES else 0))
            st = torch.zeros(shape)
            # element (row, column) of head h by the layout's rule
            h, row, col = nh - 1, dk - 1, dv - 1
            rpl = dkp // 8
            g, r = row // rpl, row % rpl
            st[h, col // 8, r * 64 + 8 * g + col % 8] = 5.0
            if mode == ops.WALK_EXP_GATES:
                st[h, 0, dkp * 8 + ((r // 4) * 8 + g) * 4 + r % 4] = 7.0
                st[h, 0, dkp * 8 + dkp] = -3.0
            S, n, m = ops.walk_state_matrices(st, dk, dv, mode)
            assert S.shape == (nh, dk, dv) and S[h, row, col] == 5.0 and S.sum() == 5.0
            if mode == ops.WALK_EXP_GATES:
                assert n[h, row] == 7.0 and n.sum() == 7.0 and m[h] == -3.0


def test_frequencies_divided_by_the_factor():
    rot = {"base": 5000.0, "dims": 6, "scaling": {"factor": 4.0}}
    want = P.frequencies(rot)
    assert want == pytest.approx([5000.0 ** (-2.0 * i / 6) / 4.0 for i in range(3)])
    got = Rotary(12, 5000.0, LinearScaling(4.0), "half", 6).frequencies()
    assert got.tolist() == pytest.approx(want, rel=1e-6)
    assert P.frequencies({"base": 5000.0, "dims": 6}) == pytest.approx([4.0 * f for f in want])


# ---------------------------------------------------------------------------
# the plain implementation against other ways of writing the same mathematics
# ---------------------------------------------------------------------------
def test_rotation_pairs_the_two_halves_of_the_leading_part():
    x = torch.randn(5, 2, 10, dtype=torch.float64)
    pos = torch.tensor([0, 1, 7, 100, 3])
    f = [0.5, 0.25, 0.125]
    y = P.rotate_halves(x, pos, f)
    assert torch.equal(y[..., 6:], x[..., 6:]) and torch.allclose(y[0], x[0])
    for t in range(5):
        for i in range(3):
            a = float(pos[t]) * f[i]
            u, v = x[t, :, i], x[t, :, i + 3]
            assert torch.allclose(y[t, :, i], u * math.cos(a) - v * math.sin(a))
            assert torch.allclose(y[t, :, i + 3], v * math.cos(a) + u * math.sin(a))
    # scores depend on the distance alone
    q, k = torch.randn(1, 1, 6, dtype=torch.float64), torch.randn(1, 1, 6, dtype=torch.float64)
    s = lambda a, b: float((P.rotate_halves(q, torch.tensor([a]), f) * P.rotate_halves(k, torch.tensor([b]), f)).sum())
    assert s(9, 4) == pytest.approx(s(25, 20))


def test_the_sink_counts_once_and_has_no_value():
    T, H, G, d, e = 9, 4, 2, 6, 5
    q, k, v = (torch.randn(T, n, w, dtype=torch.float64) for n, w in ((H, d), (G, d), (G, e)))
    sink = torch.tensor([0.3, -2.0, 1.5, 0.0], dtype=torch.float64)
    got = P.sink_attention(q, k, v, 0.4, sink)
    for h in range(H):
        for t in range(T):
            s = (k[:t + 1, h // 2] @ q[t, h]) * 0.4
            w = torch.exp(s) / (torch.exp(s).sum() + math.exp(float(sink[h])))
            assert torch.allclose(got[t, h], w @ v[:t + 1, h // 2])
    # a sink far below every score leaves the ordinary softmax; a large one takes nearly all the weight
    plain = P.sink_attention(q, k, v, 0.4, torch.full((H,), -1e9, dtype=torch.float64))
    assert torch.allclose(plain[0], v[0].repeat_interleave(2, dim=0))
    assert P.sink_attention(q, k, v, 0.4, torch.full((H,), 30.0, dtype=torch.float64)).abs().max() < 1e-6


def test_the_matrix_memory_equals_its_unrolled_sums():
    """Without the running maximum: S_t = sum_s exp(i_s + sum_(s < r <= t) f_r) k_s v_s^T; the maximum only
    rescales numerator and denominator alike, except where exp(-m) is the larger term of the denominator."""
    T, H, d, e = 12, 2, 5, 3
    q, k, v = (torch.randn(T, H, w, dtype=torch.float64) for w in (d, d, e))
    li, lf = torch.randn(T, H, dtype=torch.float64) * 3, -torch.rand(T, H, dtype=torch.float64) * 2
    got = P.matrix_memory(q, k, v, li, lf)
    for h in range(H):
        m = 0.0
        for t in range(T):
            m = max(float(lf[t, h]) + m, float(li[t, h]))
            w = torch.stack([torch.exp(li[s, h] + lf[s + 1:t + 1, h].sum()) for s in range(t + 1)])
            num = (w[:, None] * v[:t + 1, h] * (k[:t + 1, h] @ q[t, h])[:, None]).sum(0)
            nq = float((w * (k[:t + 1, h] @ q[t, h])).sum())
            den = max(abs(nq) * math.exp(-m), math.exp(-m)) + P.DENOMINATOR_FLOOR
            assert torch.allclose(got[t, h], num * math.exp(-m) / den, rtol=1e-9, atol=1e-12)


def test_the_state_space_scan_equals_its_unrolled_sums():
    T, H, G, d, e = 10, 4, 2, 3, 5
    x = torch.randn(T, H, e, dtype=torch.float64)
    B, C = torch.randn(T, G, d, dtype=torch.float64), torch.randn(T, G, d, dtype=torch.float64)
    dt = torch.rand(T, H, dtype=torch.float64) + 0.1
    A_log, D = torch.randn(H, dtype=torch.float64), torch.randn(H, dtype=torch.float64)
    got = P.state_space_scan(x, B, C, dt, A_log, D)
    for h in range(H):
        g = h // 2
        a = -math.exp(float(A_log[h]))
        for t in range(T):
            y = D[h] * x[t, h]
            for s in range(t + 1):
                y = y + math.exp(a * float(dt[s + 1:t + 1, h].sum())) * dt[s, h] * float(C[t, g] @ B[s, g]) * x[s, h]
            assert torch.allclose(got[t, h], y)


def test_the_convolutions_last_column_is_the_current_token():
    u = torch.randn(7, 3, dtype=torch.float64)
    w = torch.zeros(3, 4, dtype=torch.float64)
    w[:, -1] = 1.0
    b = torch.tensor([0.5, -1.0, 2.0], dtype=torch.float64)
    assert torch.allclose(P.biased_convolution(u, w, b), u + b)
    w[:, -1], w[:, 0] = 0.0, 1.0
    y = P.biased_convolution(u, w, b)
    assert torch.allclose(y[:3], b.expand(3, 3)) and torch.allclose(y[3:], u[:4] + b)


@pytest.mark.parametrize("name", ["odd", "wide"])
def test_a_prefix_gives_the_whole_sequences_first_logits(name):
    """Nothing looks ahead: states, convolutions, attention and the token input of a position see
    that position and earlier ones only."""
    cfg = config(name)
    g = torch.Generator().manual_seed(3)
    from sharpinference_amd.registry import build_model as bm

    specs = bm(load_config(cfg)).param_specs()
    w = {k: torch.randn(tuple(v.shape), generator=g, dtype=torch.float64) * 0.2 for k, v in specs.items()}
    toks = [int(t) for t in torch.randint(0, cfg["vocab"], (20,), generator=g)]
    layers = []
    whole = P.forward(cfg, w, toks, layers)
    assert len(layers) == len(cfg["layers"]) and whole.shape == (20, cfg["vocab"])
    assert torch.allclose(P.forward(cfg, w, toks[:13]), whole[:13], atol=1e-9)
    if cfg.get("logit_softcap"):
        assert whole.abs().max() < cfg["logit_softcap"]
    other = list(toks)
    other[5] = (other[5] + 1) % cfg["vocab"]
    changed = P.forward(cfg, w, other)
    assert torch.allclose(changed[:5], whole[:5], atol=1e-9) and not torch.allclose(changed[19], whole[19], atol=1e-6)
