"""Small Kuvonex configurations for the tests: every size differs between them and between layers."""
import copy


def _mixer(heads, dim, rot_dim, vdim, rank, scale, base, kv_from=None, dims=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale,
         "rot": {"base": base, "dims": rot_dim if dims is None else dims}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _moe(experts, top, ff, groups=None):
    router = {"experts": experts, "top": top}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def _layer(mixer, mlp):
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


# odd sizes: 3 and 5 heads, a latent of 40, a layer without a feed-forward, two shared caches,
# groups that are kept in part, a single pick, no groups
ODD = {
    "architecture": "Kuvonex", "vocab": 97, "width": 64, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.0},
    "layers": [
        _layer(_mixer(3, 24, 8, 20, 40, 0.2, 1000.0), _moe(6, 2, 40, (3, 2))),
        _layer(_mixer(5, 16, 8, 12, 40, 0.31, 1000.0, kv_from=0), None),
        _layer(_mixer(4, 32, 16, 32, 32, 0.15, 50000.0), _moe(4, 1, 24)),
        _layer(_mixer(2, 8, 16, 48, 32, 0.25, 50000.0, kv_from=2), _moe(8, 3, 16, (2, 1))),
    ],
}

# sizes the matrix-core kernels take (multiples of 16 / 32 / 128), groups of one expert each
EVEN = {
    "architecture": "Kuvonex", "vocab": 256, "width": 128, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0},
    "layers": [
        _layer(_mixer(4, 32, 32, 32, 64, 0.125, 10000.0), _moe(8, 2, 128, (8, 4))),
        _layer(_mixer(8, 16, 32, 16, 64, 0.2, 10000.0, kv_from=0), _moe(8, 8, 128)),
        _layer(_mixer(16, 64, 16, 64, 128, 0.09, 10000.0, dims=8), _moe(4, 2, 256, (2, 2))),   # half of the rotated part turns
    ],
}

# five layers of five shapes: a latent of 80 beside rows of 104 (the matrix cores take them), two caches shared
# in different ways, twelve heads over a latent of 48, one head with a rotated part of two elements, groups of
# one expert, every group kept, a width that is no multiple of 64
MID = {
    "architecture": "Kuvonex", "vocab": 211, "width": 96, "norm": {"eps": 1e-5}, "embedding": {"scale": 7.0},
    "layers": [
        _layer(_mixer(6, 40, 24, 56, 80, 0.11, 10000.0), _moe(12, 4, 80, (3, 2))),
        _layer(_mixer(2, 64, 24, 8, 80, 0.2, 10000.0, kv_from=0), _moe(5, 2, 30)),
        _layer(_mixer(4, 16, 8, 16, 48, 0.3, 300.0), None),
        _layer(_mixer(12, 32, 8, 32, 48, 0.1, 300.0, kv_from=2), _moe(9, 3, 64, (9, 9))),
        _layer(_mixer(1, 128, 2, 64, 16, 0.05, 1.0e6), _moe(2, 1, 48, (2, 1))),
    ],
}

CONFIGS = {"odd": ODD, "even": EVEN, "mid": MID}
SEEDS = {"odd": 11, "even": 12, "mid": 13}
# sinks and corrections large enough that leaving one out shows
STD_BY_SUFFIX = {".sink": 1.5, ".correction": 0.4}


def config(name):
    return copy.deepcopy(CONFIGS[name])
