"""Small Pazatar configurations for the tests: every size differs between them and between layers,
and what one has the other lacks (masks, scaling rules, convolutions, caps, feed-forwards, loops)."""
import copy


def _rot(base, dims, **scaling):
    r = {"base": base, "dims": dims}
    if scaling:
        r["scaling"] = scaling
    return r


def _attention(heads, kv_heads, dim, scale, mask=None, rot=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if mask:
        m["mask"] = {"size": mask}
    if rot:
        m["rot"] = rot
    return m


def _left(heads, kv_heads, dim, vdim, scale, mask=None, rot=None, conv=None, softcap=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if mask:
        m["mask"] = {"size": mask}
    if rot:
        m["rot"] = rot
    if conv:
        m["conv"] = conv
    if softcap:
        m["softcap"] = softcap
    return m


def _right(heads, dim, vdim, tau, rank):
    return {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "decay_rank": rank}


def _layer(kind, mixer, ff):
    return {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}


# odd sizes: head sizes no matrix-core kernel takes, values wider than keys, a chunk that is no multiple of a
# page, three taps, a loop over the middle layers only (three passes), a layer without a feed-forward, an
# attention layer that rotates a part of its heads and one that sees every key
ODD = {
    "architecture": "Pazatar", "vocab": 101, "width": 72, "norm": {"eps": 1e-5},
    "layers": [
        _layer("attention", _attention(3, 3, 10, 0.4, mask=24, rot=_rot(100.0, 6)), 40),
        _layer("parallel", {"left": _left(4, 2, 12, 20, 0.35, mask=21, rot=_rot(5000.0, 4, factor=4.0, low=1.0, high=3.0, original=64),
                                          conv=3, softcap=6.0),
                            "right": _right(2, 10, 24, 3.0, 5)}, 56),
        _layer("attention", _attention(6, 1, 8, 0.5, rot=_rot(300.0, 8, factor=6.0, original=48, fast=8.0, slow=2.0)), None),
        _layer("parallel", {"left": _left(2, 2, 16, 6, 0.3, rot=_rot(10000.0, 16), conv=2),
                            "right": _right(3, 40, 16, 1.0, 3)}, 24),
    ],
    "loop": {"start": 1, "stop": 3, "times": 3},
}

# sizes the matrix-core kernels take (heads of 64, 32 and 96, pages of 16), all layers looped twice, four taps
EVEN = {
    "architecture": "Pazatar", "vocab": 256, "width": 128, "norm": {"eps": 1e-6},
    "layers": [
        _layer("parallel", {"left": _left(4, 2, 64, 64, 0.125, mask=48, rot=_rot(20000.0, 16, factor=8.0, low=1.0, high=4.0, original=256),
                                          conv=4, softcap=20.0),
                            "right": _right(4, 32, 32, 8.0, 8)}, 256),
        _layer("attention", _attention(8, 2, 32, 0.18, mask=80, rot=_rot(10000.0, 32, factor=8.0, original=64, fast=16.0, slow=1.0)), 128),
        _layer("attention", _attention(2, 1, 96, 0.1, mask=32, rot=_rot(1000.0, 48)), 64),
    ],
    "loop": {"start": 0, "stop": 3, "times": 2},
}

# no loop at all; key channels beyond 64 and 128 (the walk's wider forms), one value column group that is not full,
# a parallel layer whose left half has neither convolution nor cap nor mask nor rotation, a single kv head, tau below 1
WIDE = {
    "architecture": "Pazatar", "vocab": 67, "width": 96, "norm": {"eps": 1e-5},
    "layers": [
        _layer("parallel", {"left": _left(4, 1, 32, 32, 0.2), "right": _right(1, 136, 20, 0.5, 2)}, 32),
        _layer("attention", _attention(4, 4, 16, 0.25, mask=16), 48),
        _layer("parallel", {"left": _left(2, 1, 24, 40, 0.2, mask=64, rot=_rot(50.0, 24), conv=8, softcap=2.0),
                            "right": _right(2, 72, 50, 16.0, 16)}, None),
    ],
    "loop": {"start": 1, "stop": 2, "times": 1},
}

CONFIGS = {"odd": ODD, "even": EVEN, "wide": WIDE}
SEEDS = {"odd": 21, "even": 22, "wide": 23}
# convolutions that mix their taps, decays spread over (0, 1), loop vectors and norm-free biases large enough to show
STD_BY_SUFFIX = {".conv": 0.6, ".a2.b": 1.5, ".a2": 1.0, ".a1": 0.3, "loop.step": 0.5}


def config(name):
    return copy.deepcopy(CONFIGS[name])


def runs_of(cfg) -> int:
    """Layer runs of a configuration (a looped layer counts each time)."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    return n if not loop else n + (loop["times"] - 1) * (loop["stop"] - loop["start"])
