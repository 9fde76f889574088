"""Small Nosedra configurations for the tests: every size differs between them and between layers,
and what one has the other lacks (rotation, its scaling, feed-forwards, the token input, the cap on
the logits, groups, taps)."""
import copy


def _left(heads, kv_heads, dim, vdim, scale, rot=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rot:
        base, dims, factor = rot
        m["rot"] = {"base": base, "dims": dims}
        if factor:
            m["rot"]["scaling"] = {"factor": factor}
    return m


def _right(heads, dim, vdim, cap):
    return {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def _parallel(left, right, ls, rs, ff):
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": ls, "right_scale": rs},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def _ssm(heads, vdim, state, groups, conv, norm_groups, ff):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                        "norm_groups": norm_groups},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


# odd sizes: head sizes no matrix-core kernel takes, values wider and narrower than keys, a rotated part narrower
# than the head, a layer without a feed-forward, two taps and four, one group and as many groups as heads, a norm in
# three parts and in one, the state-space layers first and last
ODD = {
    "architecture": "Nosedra", "vocab": 101, "width": 72, "norm": {"eps": 1e-5}, "token_side": {"dim": 5}, "logit_softcap": 9.0,
    "layers": [
        _ssm(3, 8, 10, 1, 2, 3, 40),
        _parallel(_left(4, 2, 12, 20, 0.35, rot=(5000.0, 4, 4.0)), _right(2, 10, 24, 6.0), 0.7, 1.3, 56),
        _parallel(_left(6, 1, 8, 6, 0.5, rot=(300.0, 8, None)), _right(3, 40, 16, 3.0), 1.5, 0.5, None),
        _ssm(4, 6, 20, 4, 4, 1, 24),
    ],
}

# sizes the matrix-core kernels take (heads of 64 and 32 whose values are as wide as their keys, pages of 16); the
# whole head rotated; no cap on the logits
EVEN = {
    "architecture": "Nosedra", "vocab": 256, "width": 128, "norm": {"eps": 1e-6}, "token_side": {"dim": 16},
    "layers": [
        _parallel(_left(4, 2, 64, 64, 0.125, rot=(20000.0, 64, 8.0)), _right(4, 32, 32, 12.0), 1.1, 0.8, 256),
        _ssm(8, 16, 64, 2, 4, 4, 128),
        _parallel(_left(8, 2, 32, 32, 0.18, rot=(10000.0, 16, 2.0)), _right(2, 64, 64, 8.0), 1.0, 1.0, 64),
    ],
}

# no token input and no cap; states and key channels beyond 64 and 128 (the walk's wider forms), value column groups
# that are not full, a convolution of one tap and one of eight, a left half without rotation, as many kv heads as heads
WIDE = {
    "architecture": "Nosedra", "vocab": 67, "width": 96, "norm": {"eps": 1e-5},
    "layers": [
        _parallel(_left(4, 4, 16, 16, 0.25), _right(1, 136, 20, 4.0), 1.0, 2.0, 32),
        _ssm(2, 50, 72, 1, 1, 2, 48),
        _ssm(3, 12, 136, 3, 8, 6, None),
        _parallel(_left(2, 1, 24, 40, 0.2, rot=(50.0, 24, 1.5)), _right(2, 72, 50, 1.0), 0.5, 1.0, 48),
    ],
}

CONFIGS = {"odd": ODD, "even": EVEN, "wide": WIDE}
SEEDS = {"odd": 31, "even": 32, "wide": 33}
# convolutions that mix their taps, gates and step sizes spread over their ranges, decays that are neither 0 nor 1,
# sinks, biases and norm weights large enough to show
STD_BY_SUFFIX = {".conv": 0.6, ".conv.b": 0.3, ".i": 0.5, ".f": 0.5, ".i.b": 1.0, ".f.b": 2.0, ".sink": 1.5, ".dt_bias": 1.0,
                 ".A_log": 0.7, ".D": 1.0, ".b": 0.3, "norm1": 0.3, "norm2": 0.3, "final.norm": 0.3, "side.embed": 1.0}


def config(name):
    return copy.deepcopy(CONFIGS[name])
