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

CONFIGS = {"odd": ODD, "even": EVEN}
SEEDS = {"odd": 11, "even": 12}
# sinks and corrections large enough that leaving one out shows
STD_BY_SUFFIX = {".sink": 1.5, ".correction": 0.4}


def config(name):
    return copy.deepcopy(CONFIGS[name])
