"""Small Fovosun configurations for the tests: every size differs between them and between layers,
and what one has the other lacks (streams, rotation, windows, convolutions, the query temperature,
feed-forwards, shared experts)."""
import copy


def _diff(kind, heads, kv_heads, dim, vdim, scale, diff, rot=None, window=None, conv=None, q_temp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff}
    if rot:
        m["rot"] = {"base": rot[0], "dims": rot[1]}
    if window:
        m["mask"] = {"size": window}
    if conv:
        m["conv"] = conv
    if q_temp:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return {"type": kind, "mixer": m}


def _ret(heads, dim, vdim, decay, rot=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}
    if rot:
        m["rot"] = {"base": rot[0], "dims": rot[1]}
    return {"type": "retention", "mixer": m}


def _dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def _moe(experts, top, ff, limit, shared=None):
    m = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared[0], "limit": shared[1]}
    return m


def _layer(mixer, mlp):
    return {**mixer, "mlp": mlp}


# odd sizes: head sizes no matrix-core kernel takes, values wider and narrower than a head's two maps, a rotated part
# narrower than a map, windows that are no multiple of a page, two streams, a layer without a feed-forward, one
# pick and three, an attention_2 layer without window and rotation, as many kv heads as heads
ODD = {
    "architecture": "Fovosun", "vocab": 101, "width": 72, "norm": {"eps": 1e-5}, "embedding": {"scale": 2.5}, "streams": 2,
    "layers": [
        _layer(_diff("attention_2", 4, 2, 12, 20, 0.35, 0.2, rot=(5000.0, 8), window=37), _dense(40, 1.2)),
        _layer(_ret(3, 10, 24, (0.9, 0.97, 0.995), rot=(300.0, 6)), None),
        _layer(_diff("attention", 6, 1, 8, 6, 0.5, 0.45, conv=2, q_temp=(0.4, 16)), _moe(5, 3, 24, 0.9, shared=(16, 1.4))),
        _layer(_diff("attention_2", 3, 3, 10, 33, 0.3, 0.1), _moe(4, 1, 20, 2.5)),
    ],
}

# sizes the matrix-core kernels take (a head's two maps of 32 + 32 or 64 + 64 elements with values as wide, pages of
# 16, widths that are multiples of 128); four streams; a shared expert of the experts' own width and limit (it rides
# with the routed ones), and one of another width; the whole map rotated
EVEN = {
    "architecture": "Fovosun", "vocab": 256, "width": 128, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0}, "streams": 4,
    "layers": [
        _layer(_diff("attention", 4, 2, 32, 64, 0.18, 0.3, conv=4, q_temp=(0.25, 32)), _moe(8, 2, 128, 1.5, shared=(128, 1.5))),
        _layer(_diff("attention_2", 8, 2, 32, 64, 0.2, 0.25, rot=(20000.0, 32), window=48), _dense(256, 2.0)),
        _layer(_ret(2, 64, 64, (0.96875, 0.9990234375), rot=(10000.0, 32)), _moe(6, 2, 128, 1.0, shared=(256, 3.0))),
        _layer(_diff("attention_2", 2, 1, 64, 128, 0.125, 0.35, rot=(100.0, 16), window=100), _dense(128, 0.7)),
    ],
}

# one plain residual sum (no streams); key channels beyond 64 and 128 in the retention (the walk's wider forms), a
# retention without rotation, eight taps, a window of one page, every expert picked
WIDE = {
    "architecture": "Fovosun", "vocab": 67, "width": 96, "norm": {"eps": 1e-5}, "embedding": {"scale": 4.0},
    "layers": [
        _layer(_ret(1, 136, 20, (0.98,)), _dense(48, 1.0)),
        _layer(_diff("attention", 2, 2, 24, 40, 0.2, 0.5, conv=8), _moe(3, 3, 32, 1.3)),
        _layer(_diff("attention_2", 4, 1, 16, 16, 0.25, 0.3, rot=(50.0, 16), window=16), None),
        _layer(_ret(2, 72, 50, (1.0, 0.9), rot=(1000.0, 72)), _moe(2, 1, 16, 0.8, shared=(24, 0.6))),
    ],
}

# one stream kept the way several are; score maps of 136 elements (a head's two maps are wider than any value row)
ONE = {
    "architecture": "Fovosun", "vocab": 50, "width": 64, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.5}, "streams": 1,
    "layers": [
        _layer(_diff("attention", 2, 1, 136, 32, 0.09, 0.2, q_temp=(0.5, 8)), _dense(32, 1.0)),
        _layer(_ret(2, 16, 8, (0.9, 0.99), rot=(100.0, 16)), _moe(4, 2, 16, 1.0)),
    ],
}

CONFIGS = {"odd": ODD, "even": EVEN, "wide": WIDE, "one": ONE}
SEEDS = {"odd": 41, "even": 42, "wide": 43, "one": 44}
# convolutions that mix their taps, stream weights of order one, lambdas away from their constant, biases and norm
# weights large enough to show
STD_BY_SUFFIX = {".conv": 0.6, ".b": 0.3, ".in": 0.7, ".out": 0.7, ".mix": 0.6, ".lq1": 0.35, ".lk1": 0.35, ".lq2": 0.35, ".lk2": 0.35,
                 "norm1": 0.3, "norm2": 0.3, "final.norm": 0.3, ".g": 0.3}


def config(name):
    return copy.deepcopy(CONFIGS[name])
