"""Fovosun without a GPU: the configuration reader, the tensors the model asks for, the memory each
layer gets, and the plain implementation's own consistency (what the GPU tests lean on)."""
import math

import pytest
import torch

import plain_fovosun as P
from tiny_fovosun import CONFIGS, config

from sharpinference_amd import load_config
from sharpinference_amd.cache.spec import WINDOW_NONE, WINDOW_SLIDING, KVSpec, StateSpec, kv_of, states_of
from sharpinference_amd.config.base import ConfigError
from sharpinference_amd.config.fovosun import FovosunConfig
from sharpinference_amd.parts.block import HyperBlock, PreNormBlock
from sharpinference_amd.registry import build_model, registered_architectures


def test_the_design_is_registered_and_its_configuration_round_trips():
    assert "Fovosun" in registered_architectures()
    for name in CONFIGS:
        cfg = load_config(config(name))
        assert isinstance(cfg, FovosunConfig)
        assert cfg.to_dict() == config(name)
        assert load_config(cfg.to_dict()) == cfg


def test_what_the_file_leaves_out_is_off():
    cfg = load_config(config("odd"))
    a2, ret, att, bare = (l.mixer for l in cfg.layers)
    assert a2.conv is None and a2.q_temp is None and a2.window == 37 and a2.rot.dims == 8
    assert att.rot is None and att.window is None and att.conv == 2 and att.q_temp == (0.4, 16.0)
    assert bare.rot is None and bare.window is None
    assert cfg.layers[1].mlp is None and cfg.layers[3].mlp.shared_ff == 0 and cfg.layers[2].mlp.shared_ff == 16
    assert load_config(config("wide")).streams is None
    assert all(isinstance(b, PreNormBlock) and not isinstance(b, HyperBlock) for b in build_model(load_config(config("wide"))).blocks)
    assert all(isinstance(b, HyperBlock) for b in build_model(load_config(config("one"))).blocks)
    d = config("odd")
    d["layers"][0]["mixer"].pop("kv_heads"), d["layers"][0]["mixer"].pop("vdim"), d["layers"][0]["mixer"].pop("scale")
    m = load_config(d).layers[0].mixer
    assert (m.kv_heads, m.vdim) == (4, 12) and m.scale == pytest.approx(12 ** -0.5)


@pytest.mark.parametrize("path, value, what", [
    (("layers", 0, "mixer", "sink"), 1.0, "sink"),
    (("layers", 0, "mixer", "rot", "scaling"), {"factor": 2.0}, "scaling"),
    (("layers", 0, "mixer", "mask", "kind"), "chunk", "kind"),
    (("layers", 1, "mixer", "gate_cap"), 2.0, "gate_cap"),
    (("layers", 2, "mixer", "q_temp", "base"), 2.0, "base"),
    (("layers", 2, "mlp", "router", "groups"), 2, "groups"),
    (("layers", 2, "mlp", "shared", "count"), 2, "count"),
    (("layers", 0, "mlp", "bias"), True, "bias"),
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
    (lambda d: d["layers"][0]["mixer"].update(kv_heads=3), "kv heads"),
    (lambda d: d["layers"][0]["mixer"].update(dim=11), "dim"),
    (lambda d: d["layers"][0]["mixer"]["rot"].update(dims=14), "dims"),
    (lambda d: d["layers"][0]["mixer"].update(diff=1.0), "diff"),
    (lambda d: d["layers"][0]["mixer"].update(conv=3), "conv"),
    (lambda d: d["layers"][0]["mixer"]["mask"].update(size=0), "size"),
    (lambda d: d["layers"][1]["mixer"].update(decay=[0.5, 0.6]), "decay"),
    (lambda d: d["layers"][1]["mixer"].update(decay=[0.5, 0.6, 1.5]), "decay"),
    (lambda d: d["layers"][2]["mixer"].update(conv=1), "conv"),
    (lambda d: d["layers"][2]["mlp"]["router"].update(top=6), "top"),
    (lambda d: d["layers"][2]["mlp"]["expert"].update(limit=0.0), "limit"),
    (lambda d: d["layers"][0].update(type="mamba2"), "mamba2"),
    (lambda d: d["layers"][0]["mlp"].update(kind="gated"), "kind"),
    (lambda d: d.update(streams=9), "streams"),
    (lambda d: d.update(vocab=0), "vocab"),
])
def test_sizes_that_contradict_each_other_are_refused(change, what):
    d = config("odd")
    change(d)
    with pytest.raises(ConfigError, match=what):
        load_config(d)


def _expected_tensors(d):
    W, S = d["width"], d.get("streams")
    out = {"embed": (d["vocab"], W), "head": (d["vocab"], W), "final.norm": (W,)}
    for i, layer in enumerate(d["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (W,)
        if S:
            out.update({p + "hc1.in": (S,), p + "hc1.out": (S,), p + "hc1.mix": (S, S)})
        if layer["type"] == "retention":
            qk, vv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            out.update({p + "mix.q": (qk, W), p + "mix.k": (qk, W), p + "mix.v": (vv, W), p + "mix.g": (vv, W), p + "mix.o": (W, vv)})
        else:
            q, k, v = m["heads"] * 2 * m["dim"], m["kv_heads"] * 2 * m["dim"], m["kv_heads"] * m["vdim"]
            out.update({p + "mix.q": (q, W), p + "mix.k": (k, W), p + "mix.v": (v, W), p + "mix.o": (W, m["heads"] * m["vdim"])})
            out.update({p + "mix." + n: (m["dim"],) for n in ("lq1", "lk1", "lq2", "lk2")})
            if layer["type"] == "attention_2":
                out.update({p + "mix.q.b": (q,), p + "mix.k.b": (k,), p + "mix.v.b": (v,)})
            else:
                out[p + "mix.g"] = (m["heads"], W)
            if m.get("conv"):
                out.update({p + "mix.q.conv": (q, m["conv"]), p + "mix.k.conv": (k, m["conv"]), p + "mix.v.conv": (v, m["conv"])})
        f = layer["mlp"]
        if f is None:
            continue
        out[p + "norm2"] = (W,)
        if S:
            out.update({p + "hc2.in": (S,), p + "hc2.out": (S,), p + "hc2.mix": (S, S)})
        if f["kind"] == "dense":
            out.update({p + "mlp.gate": (f["ff"], W), p + "mlp.up": (f["ff"], W), p + "mlp.down": (W, f["ff"])})
        else:
            E, ff = f["router"]["experts"], f["expert"]["ff"]
            out.update({p + "mlp.router": (E, W), p + "mlp.router.b": (E,)})
            for e in range(E):
                out.update({f"{p}mlp.e{e}.gate": (ff, W), f"{p}mlp.e{e}.up": (ff, W), f"{p}mlp.e{e}.down": (W, ff)})
            if f.get("shared"):
                sf = f["shared"]["ff"]
                out.update({p + "mlp.shared.gate": (sf, W), p + "mlp.shared.up": (sf, W), p + "mlp.shared.down": (W, sf)})
    return out


@pytest.mark.parametrize("name", list(CONFIGS))
def test_the_model_asks_for_the_designs_tensors_by_name_and_shape(name):
    specs = build_model(load_config(config(name))).param_specs()
    want = _expected_tensors(config(name))
    assert set(specs) == set(want)
    assert {n: tuple(s.shape) for n, s in specs.items()} == want


def test_the_memory_every_layer_gets():
    from sharpinference_amd import ops

    specs = build_model(load_config(config("odd"))).cache_specs()
    assert specs[0] == KVSpec(2, 24, WINDOW_SLIDING, 37, 20)                 # a key head's two maps are one row of 2 x 12
    assert specs[1] == StateSpec(ops.walk_state_shape(3, 10, 24, ops.WALK_FIXED_DECAY), torch.float32)
    assert kv_of(specs[2]) == KVSpec(1, 16, WINDOW_NONE, 0, 6)
    assert states_of(specs[2]) == (StateSpec((1, 6 * 16 + 16 + 6), torch.float32),)     # the last tap - 1 rows of q | k | v
    assert specs[3] == KVSpec(3, 20, WINDOW_NONE, 0, 33)
    even = build_model(load_config(config("even"))).cache_specs()
    assert kv_of(even[0]) == KVSpec(2, 64, WINDOW_NONE, 0, 0) and even[1] == KVSpec(2, 64, WINDOW_SLIDING, 48, 0)


# ---------------------------------------------------------------------------
# the plain implementation's own identities
# ---------------------------------------------------------------------------
def test_retention_is_its_unrolled_sum_and_carries_its_state():
    g = torch.Generator().manual_seed(1)
    W, m = 20, {"heads": 2, "dim": 6, "vdim": 4, "decay": [0.9, 0.5], "rot": {"base": 50.0, "dims": 4}}
    w = {"p." + n: torch.randn(s, W, generator=g, dtype=torch.float64) * 0.3 for n, s in (("q", 12), ("k", 12), ("v", 8), ("g", 8))}
    w["p.o"] = torch.randn(W, 8, generator=g, dtype=torch.float64) * 0.3
    h = torch.randn(9, W, generator=g, dtype=torch.float64)
    whole, S = P.retention(h, w, "p.", m, 1e-6)
    first, S1 = P.retention(h[:5], w, "p.", m, 1e-6)
    rest, S2 = P.retention(h[5:], w, "p.", m, 1e-6, state=S1, first_position=5)
    assert torch.allclose(torch.cat([first, rest]), whole, atol=1e-12) and torch.allclose(S2, S, atol=1e-12)
    # o_t = sum_(s <= t) decay^(t - s) (q_t . k_s) v_s, q and k rotated, k scaled
    pos = torch.arange(9)
    q = P.rotate_half_split((h @ w["p.q"].T).reshape(9, 2, 6), pos, 50.0, 4)
    k = P.rotate_half_split((h @ w["p.k"].T).reshape(9, 2, 6), pos, 50.0, 4) * 6 ** -0.5
    v = (h @ w["p.v"].T).reshape(9, 2, 4)
    o = torch.zeros(9, 2, 4, dtype=torch.float64)
    for t in range(9):
        for s in range(t + 1):
            for hh in range(2):
                o[t, hh] += m["decay"][hh] ** (t - s) * (q[t, hh] @ k[s, hh]) * v[s, hh]
    want = (P.unit_rms(o, 1e-6).reshape(9, 8) * P.silu(h @ w["p.g"].T)) @ w["p.o"].T
    assert torch.allclose(whole, want, atol=1e-10)


def test_a_rotation_depends_on_the_distance_alone_and_leaves_the_rest_of_a_head():
    g = torch.Generator().manual_seed(2)
    x, y = torch.randn(1, 1, 10, generator=g, dtype=torch.float64), torch.randn(1, 1, 10, generator=g, dtype=torch.float64)
    def score(p, q):
        a = P.rotate_half_split(x, torch.tensor([p]), 100.0, 6)
        b = P.rotate_half_split(y, torch.tensor([q]), 100.0, 6)
        return float((a * b).sum())
    assert score(7, 3) == pytest.approx(score(104, 100), abs=1e-9)
    assert torch.equal(P.rotate_half_split(x, torch.tensor([5]), 100.0, 6)[..., 6:], x[..., 6:])
    a = P.rotate_half_split(x, torch.tensor([1]), 100.0, 6)[0, 0]
    f1 = 100.0 ** (-2.0 / 6)
    assert float(a[1]) == pytest.approx(float(x[0, 0, 1] * math.cos(f1) - x[0, 0, 4] * math.sin(f1)), abs=1e-12)


def test_the_window_keeps_itself_and_the_tokens_before_it():
    m = P.visible(9, 3)
    assert m[5].tolist() == [False, False, False, True, True, True, False, False, False]
    assert P.visible(4, None)[3].all() and not P.visible(4, None)[0, 1]


def test_the_convolutions_last_tap_is_the_current_token_and_zeros_stand_before_the_first():
    u = torch.arange(12, dtype=torch.float64).reshape(6, 2) + 1.0
    w = torch.tensor([[0.0, 0.0, 1.0], [1.0, 0.0, 0.0]], dtype=torch.float64)
    y = P.causal_conv(u, w)
    assert torch.equal(y[:, 0], u[:, 0]) and y[:2, 1].tolist() == [0.0, 0.0] and torch.equal(y[2:, 1], u[:4, 1])


def test_the_difference_of_two_equal_maps_and_the_temperatures_steps():
    a = torch.randn(3, 2, 8, dtype=torch.float64)
    o = P.difference_of_maps(a, a, 0.25, 0.4, 0.0)
    assert torch.allclose(o, P.unit_rms(a, 0.0) * 0.6, atol=1e-12)           # (1 - lambda) a, normed: the scale falls out
    w = {"p.lq1": torch.tensor([1.0, 2.0]), "p.lk1": torch.tensor([0.5, 0.0]), "p.lq2": torch.tensor([0.0, 1.0]), "p.lk2": torch.tensor([3.0, -1.0])}
    assert float(P.difference_lambda(w, "p.", 0.3)) == pytest.approx(math.exp(0.5) - math.exp(-1.0) + 0.3)
    t = P.query_temperature(torch.tensor([0, 6, 7, 14, 15]), 0.5, 8.0, torch.float64)
    assert t.tolist() == pytest.approx([1.0, 1.0, 1.0 + 0.5 * math.log(2.0), 1.0 + 0.5 * math.log(2.0), 1.0 + 0.5 * math.log(3.0)])


def test_a_query_with_the_other_maps_place_zeroed_scores_its_own_map():
    """What the engine's attention kernels are given: a head's two maps as one key row, and one query
    row per map with zeros in the other map's place."""
    g = torch.Generator().manual_seed(3)
    q, k = torch.randn(5, 2, 6, generator=g, dtype=torch.float64), torch.randn(5, 2, 6, generator=g, dtype=torch.float64)
    for mp in range(2):
        wide = torch.zeros(5, 12, dtype=torch.float64)
        wide[:, mp * 6:(mp + 1) * 6] = q[:, mp]
        assert torch.allclose(wide @ k.reshape(5, 12).T, q[:, mp] @ k[:, mp].T, atol=1e-14)


def test_the_clamped_unit_the_routers_choice_and_the_streams():
    w = {"p.gate": torch.eye(3, dtype=torch.float64), "p.up": torch.eye(3, dtype=torch.float64), "p.down": torch.eye(3, dtype=torch.float64)}
    h = torch.tensor([[5.0, -5.0, 0.5]], dtype=torch.float64)
    y = P.clamped_glu(h, w, "p.", 2.0)[0]
    sig = lambda z: 1.0 / (1.0 + math.exp(-z))
    assert y.tolist() == pytest.approx([2.0 * sig(1.702 * 2.0) * 3.0, -5.0 * sig(-1.702 * 5.0) * (-2.0 + 1.0), 0.5 * sig(1.702 * 0.5) * 1.5])
    wr = {"p.router": torch.eye(4, dtype=torch.float64), "p.router.b": torch.tensor([0.0, 0.0, 0.0, 2.5], dtype=torch.float64)}
    idx, wts = P.router_choice(torch.tensor([[1.0, 3.0, 2.0, 0.0]], dtype=torch.float64), wr, "p.", 2)
    assert idx.tolist() == [[1, 3]] and wts[0].tolist() == pytest.approx([sig(0.5), 1.0 - sig(0.5)])
    xs = torch.randn(3, 4, 5, dtype=torch.float64)
    y = torch.randn(4, 5, dtype=torch.float64)
    new = P.streams_write(xs, y, torch.eye(3, dtype=torch.float64), torch.ones(3, dtype=torch.float64))
    assert torch.allclose(new, xs + y[None])                                   # an identity mix is the plain residual sum
    mix = torch.zeros(3, 3, dtype=torch.float64)
    mix[0, 2] = 1.0                                                             # stream 0 goes to stream 2: [from, to]
    new = P.streams_write(xs, y, mix, torch.zeros(3, dtype=torch.float64))
    assert torch.equal(new[2], xs[0]) and not new[0].any() and not new[1].any()
    assert torch.allclose(P.streams_read(xs, torch.tensor([1.0, 0.0, -2.0], dtype=torch.float64)), xs[0] - 2.0 * xs[2])


def test_a_prefixs_logits_are_the_whole_sequences_first():
    from sharpinference_amd.weights.loader import write_random_model
    import tempfile
    from tiny_fovosun import SEEDS, STD_BY_SUFFIX

    with tempfile.TemporaryDirectory() as d:
        write_random_model(load_config(config("odd")), d, SEEDS["odd"], std=0.1, std_by_suffix=STD_BY_SUFFIX)
        cfg, w = P.read_config(d), P.load_weights(d)
        toks = [(7 * i + 3) % 101 for i in range(50)]
        whole = P.forward(cfg, w, toks)
        assert torch.allclose(P.forward(cfg, w, toks[:21]), whole[:21], atol=1e-9)
        lo = []
        P.forward(cfg, w, toks[:5], layer_outputs=lo)
        assert len(lo) == 4 and all(x.shape == (5, 72) for x in lo)
