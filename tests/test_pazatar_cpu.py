"""Pazatar without a GPU: the configuration reader, the tensors the model asks for, the order its
layers run in and the memory each run gets, the frequency tables, and the plain implementation's
own consistency (what the GPU tests lean on)."""
import copy
import math

import pytest
import torch

import plain_pazatar as P
from tiny_pazatar import CONFIGS, config, runs_of

from sharpinference_amd import load_config
from sharpinference_amd.cache.manager import CacheManager
from sharpinference_amd.cache.spec import KVSpec, MixedSpec, StateSpec, combine_specs, kv_of, states_of
from sharpinference_amd.config.base import ConfigError
from sharpinference_amd.config.pazatar import DEFAULT_DECAY_RANK, PazatarConfig
from sharpinference_amd.parts.position import Rotary, WavelengthScaling, YarnRotary, YarnScaling
from sharpinference_amd.registry import build_model, registered_architectures


def test_the_design_is_registered_and_its_configuration_round_trips():
    assert "Pazatar" in registered_architectures()
    for name in CONFIGS:
        cfg = load_config(config(name))
        assert isinstance(cfg, PazatarConfig)
        again = load_config(cfg.to_dict())
        # what to_dict leaves out is the size that a tensor's shape gives
        strip = lambda c: [(l.type, l.attention, None if l.linear is None else (l.linear.heads, l.linear.dim, l.linear.vdim, l.linear.tau), l.ff)
                           for l in c.layers]
        assert strip(again) == strip(cfg) and (again.loop_start, again.loop_stop, again.loop_times) == (cfg.loop_start, cfg.loop_stop, cfg.loop_times)


@pytest.mark.parametrize("path, value, what", [
    (("layers", 0, "mixer", "window"), 7, "window"),
    (("layers", 1, "mixer", "left", "rot", "scaling", "fast"), 2.0, "fast"),           # a YaRN key in the stretched rule
    (("layers", 2, "mixer", "rot", "scaling", "low"), 1.0, "low"),                      # and the other way round
    (("layers", 0, "mixer", "softcap"), 5.0, "softcap"),                                 # the attention layer has no cap
    (("loop", "step"), 1, "step"),
    (("norm", "kind"), "layer", "kind"),
    (("bias",), True, "bias"),
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
    (lambda d: d["loop"].update(stop=5), "loop"),
    (lambda d: d["loop"].update(start=3, stop=3), "loop"),
    (lambda d: d["layers"][0]["mixer"].update(kv_heads=2), "kv_heads"),
    (lambda d: d["layers"][0]["mixer"].update(vdim=12), "vdim"),
    (lambda d: d["layers"][1]["mixer"]["left"].update(conv=1), "conv"),
    (lambda d: d["layers"][1]["mixer"]["left"]["rot"].update(dims=14), "dims"),
    (lambda d: d["layers"][1]["mixer"]["right"].update(tau=0.0), "tau"),
    (lambda d: d["layers"][0].update(type="recurrent"), "recurrent"),
    (lambda d: d["layers"][0]["mlp"].update(kind="moe"), "kind"),
])
def test_contradictions_are_refused(change, what):
    d = config("odd")
    change(d)
    with pytest.raises(ConfigError, match=what):
        load_config(d)


def test_options_a_layer_leaves_out_are_off():
    d = config("wide")
    cfg = load_config(d)
    left = cfg.layers[0].attention
    assert (left.mask_size, left.rot, left.softcap, left.conv) == (0, None, 0.0, 0)
    model = build_model(cfg)
    mixer = model.blocks[0].mixer.branches[0][1]
    assert mixer.rotary is None and mixer.conv_taps == 0 and mixer.softcap == 0.0 and mixer.sink and mixer.window_kind == 0
    assert isinstance(mixer.cache_spec(), KVSpec)                       # no convolution: no state beside the pages
    del d["loop"]
    model = build_model(load_config(d))
    assert "loop.step" not in model.param_specs() and all(r.add_row is None for r in model.schedule)


def test_tensor_names_and_shapes():
    cfg = load_config(config("odd"))
    specs = build_model(cfg).param_specs()
    W = 72
    want = {
        "embed": (101, W), "final.norm": (W,), "loop.step": (3, W),
        "l0.norm1": (W,), "l0.norm1b": (W,), "l0.norm2": (W,), "l0.norm2b": (W,),
        "l0.mix.q": (30, W), "l0.mix.k": (30, W), "l0.mix.q.norm": (30,), "l0.mix.k.norm": (30,), "l0.mix.o": (W, 30),
        "l0.mlp.up": (40, W), "l0.mlp.down": (W, 40),
        "l1.mix.left.q": (48, W), "l1.mix.left.k": (24, W), "l1.mix.left.v": (40, W), "l1.mix.left.o": (W, 80),
        "l1.mix.left.q.norm": (12,), "l1.mix.left.k.norm": (12,),
        "l1.mix.left.q.conv": (48, 3), "l1.mix.left.k.conv": (24, 3), "l1.mix.left.v.conv": (40, 3),
        "l1.mix.left.out": (W,), "l1.mix.right.out": (W,),
        "l1.mix.right.q": (20, W), "l1.mix.right.k": (20, W), "l1.mix.right.v": (48, W), "l1.mix.right.g": (48, W),
        "l1.mix.right.o": (W, 48), "l1.mix.right.norm": (24,), "l1.mix.right.a1": (5, W), "l1.mix.right.a2": (20, 5),
        "l1.mix.right.a2.b": (20,),
    }
    for name, shape in want.items():
        assert name in specs and tuple(specs[name].shape) == shape, name
    assert not any(n.startswith("l2.mlp.") or n.startswith("l2.norm2") for n in specs)       # layer 2 has no feed-forward
    assert "l2.mix.v" not in specs and "head" not in specs and "lm_head.weight" not in specs  # values are keys; the head is the table
    assert "l3.mix.left.v.conv" in specs and tuple(specs["l3.mix.left.v.conv"].shape) == (12, 2)


def test_the_decay_projection_takes_its_rank_from_the_tensor():
    d = config("odd")
    del d["layers"][1]["mixer"]["right"]["decay_rank"]
    cfg = load_config(d)
    assert cfg.layers[1].linear.decay_rank is None
    assert tuple(build_model(cfg).param_specs()["l1.mix.right.a1"].shape) == (DEFAULT_DECAY_RANK, 72)
    seen = cfg.with_tensor_shapes({"l1.mix.right.a1": ((11, 72), torch.bfloat16), "l3.mix.right.a1": ((2, 72), torch.bfloat16)})
    assert seen.layers[1].linear.decay_rank == 11 and seen.layers[3].linear.decay_rank == 3      # a given rank stays
    assert tuple(build_model(seen).param_specs()["l1.mix.right.a2"].shape) == (20, 11)
    assert "decay_rank" not in str(seen.to_dict())


def test_every_pass_of_the_loop_has_memory_of_its_own():
    for name in CONFIGS:
        d = config(name)
        model = build_model(load_config(d))
        order = P.layer_order(d)
        assert [r.layer for r in model.schedule] == [i for i, _ in order] and len(order) == runs_of(d)
        assert [r.cache for r in model.schedule] == list(range(len(order)))                  # no slot is shared
        loop = d["loop"]
        for r, (i, t) in zip(model.schedule, order):
            assert r.add_row == (("loop.step", t) if t is not None and i == loop["start"] else None)
        specs = model.cache_specs()
        for r, spec in zip(model.schedule, specs):
            layer = d["layers"][r.layer]
            if layer["type"] == "attention":
                assert isinstance(spec, KVSpec)
                continue
            left, right = layer["mixer"]["left"], layer["mixer"]["right"]
            states = states_of(spec)
            assert kv_of(spec).head_dim == left["dim"] and kv_of(spec).value_dim == left["vdim"]
            rows = next(n for n in (32, 64, 128, 256) if right["dim"] <= n)                  # (what the walk's lanes cover)
            assert states[-1].shape == (right["heads"], -(-right["vdim"] // 8), rows, 8) and states[-1].dtype == torch.float32
            if left.get("conv"):
                channels = left["heads"] * left["dim"] + left["kv_heads"] * (left["dim"] + left["vdim"])
                assert len(states) == 2 and states[0].shape == (left["conv"] - 1, channels)
            else:
                assert len(states) == 1


def test_the_cache_manager_keeps_states_beside_pages():
    kv = KVSpec(2, 16, 1, 32)
    a, b = StateSpec((3, 5)), StateSpec((2, 4, 6))
    assert combine_specs([kv, None]) == kv and combine_specs([None, b]) == b and combine_specs([None]) is None
    mixed = combine_specs([MixedSpec(kv, (a,)), b])
    assert mixed == MixedSpec(kv, (a, b))
    with pytest.raises(ValueError):
        combine_specs([kv, KVSpec(1, 8)])
    cm = CacheManager([mixed, b, kv, None], 16, 8, 2, torch.float32, "cpu")
    assert [len(s) for s in cm.states] == [2, 1, 0, 0] and cm.states[0][1].shape == (3, 2, 4, 6) and cm.state[0] is cm.states[0][0]
    assert cm.k[0] is not None and cm.k[1] is None and cm.k[2] is not None and len(cm.groups) == 1
    cm.add_request("x")
    slot = cm.requests["x"].state_slot
    for per in cm.states:
        for t in per:
            t[slot].fill_(7.0)
    cm.free_request("x")
    cm.add_request("y")                                        # the slot comes back, and comes back zeroed
    assert cm.requests["y"].state_slot == slot
    assert all(float(t[slot].abs().max()) == 0.0 for per in cm.states for t in per)
    cm.check_invariants()


# ----------------------------------------------------------------------------
# frequency tables: the package's against the plain implementation's
# ----------------------------------------------------------------------------
@pytest.mark.parametrize("base, dims, s", [(10000.0, 96, dict(factor=8.0, original=512, fast=32.0, slow=1.0)),
                                           (300.0, 8, dict(factor=6.0, original=48, fast=8.0, slow=2.0)),
                                           (1000.0, 64, dict(factor=2.0, original=4096, fast=1.5, slow=1.4)),
                                           (50.0, 6, dict(factor=3.0, original=8, fast=64.0, slow=0.01))])
def test_yarn_frequencies_and_magnitude(base, dims, s):
    rot = YarnRotary(dims + 4, base, YarnScaling(s["factor"], s["original"], s["fast"], s["slow"]), "interleaved", dims)
    want = torch.tensor(P.yarn_frequencies(base, dims, s), dtype=torch.float64)
    assert torch.allclose(rot.frequencies().double(), want, rtol=1e-6, atol=0)
    assert abs(rot.magnitude - (0.1 * math.log(s["factor"]) + 1.0)) < 1e-12 and abs(P.yarn_magnitude(s) - rot.magnitude) < 1e-12
    plain = torch.tensor(P.plain_frequencies(base, dims), dtype=torch.float64)
    assert (want <= plain * (1 + 1e-12)).all() and (want >= plain / s["factor"] * (1 - 1e-12)).all()


@pytest.mark.parametrize("base, dims, s", [(20000.0, 24, dict(factor=8.0, low=1.0, high=4.0, original=2048)),
                                           (5000.0, 4, dict(factor=4.0, low=1.0, high=3.0, original=64)),
                                           (100.0, 32, dict(factor=16.0, low=0.5, high=8.0, original=100))])
def test_stretched_wavelengths(base, dims, s):
    rot = Rotary(dims, base, WavelengthScaling(s["factor"], s["low"], s["high"], s["original"]), "half", dims)
    want = torch.tensor(P.stretched_frequencies(base, dims, s), dtype=torch.float64)
    assert torch.allclose(rot.frequencies().double(), want, rtol=1e-6, atol=0)
    kinds = {round(float(w / p), 6) for w, p in zip(want, torch.tensor(P.plain_frequencies(base, dims), dtype=torch.float64))}
    assert len(kinds) > 1                                      # the rule does something at these sizes


# ----------------------------------------------------------------------------
# the plain implementation's own consistency
# ----------------------------------------------------------------------------
def test_the_recurrence_carried_in_a_state_equals_the_recurrence_from_the_start():
    g = torch.Generator().manual_seed(1)
    T, H, d, e = 23, 2, 5, 7
    q, k = torch.randn(T, H, d, generator=g, dtype=torch.float64), torch.randn(T, H, d, generator=g, dtype=torch.float64)
    v = torch.randn(T, H, e, generator=g, dtype=torch.float64)
    alpha = torch.rand(T, H, d, generator=g, dtype=torch.float64)
    whole = P.gated_recurrence(q, k, v, alpha)
    # the state after 9 tokens, written out: sum over s <= t of (prod of later decays) k_s v_s^T
    S = torch.zeros(H, d, e, dtype=torch.float64)
    for s in range(9):
        S += torch.prod(alpha[s + 1:9], dim=0)[:, :, None] * k[s][:, :, None] * v[s][:, None, :]
    rest = P.gated_recurrence(q[9:], k[9:], v[9:], alpha[9:], state=S)
    assert torch.allclose(rest, whole[9:], rtol=1e-10, atol=1e-12)
    # decays of one: plain (unnormalised) linear attention
    ones = P.gated_recurrence(q, k, v, torch.ones_like(alpha))
    scores = torch.einsum("thd,shd->hts", q, k) * torch.tril(torch.ones(T, T, dtype=torch.float64))
    assert torch.allclose(ones, torch.einsum("hts,she->the", scores, v), rtol=1e-10, atol=1e-12)


def test_the_convolution_starts_from_zeros_and_looks_only_back():
    g = torch.Generator().manual_seed(2)
    u, w = torch.randn(9, 4, generator=g, dtype=torch.float64), torch.randn(4, 3, generator=g, dtype=torch.float64)
    y = P.short_convolution(u, w)
    assert torch.allclose(y[0], w[:, 2] * u[0]) and torch.allclose(y[1], w[:, 1] * u[0] + w[:, 2] * u[1])
    assert torch.allclose(y[5], w[:, 0] * u[3] + w[:, 1] * u[4] + w[:, 2] * u[5])
    u2 = u.clone()
    u2[6:] += 1.0
    assert torch.equal(P.short_convolution(u2, w)[:6], y[:6])


def test_chunks_are_counted_from_the_sequences_start_and_the_sink_takes_its_share():
    pos = torch.arange(10)
    m = P.visible(pos, 4)
    assert m[3].tolist() == [True] * 4 + [False] * 6 and m[4].tolist() == [False] * 4 + [True] + [False] * 5
    assert m[9].tolist() == [False] * 8 + [True] * 2 and P.visible(pos, None)[9].all()
    q, k, v = torch.zeros(10, 1, 2, dtype=torch.float64), torch.zeros(10, 1, 2, dtype=torch.float64), torch.ones(10, 1, 3, dtype=torch.float64)
    out = P.masked_attention(q, k, v, m, 1.0, sink=True)       # all scores 0: n keys and the sink share the weight
    assert torch.allclose(out[:, 0, 0], torch.tensor([1 / 2, 2 / 3, 3 / 4, 4 / 5, 1 / 2, 2 / 3, 3 / 4, 4 / 5, 1 / 2, 2 / 3], dtype=torch.float64))
    big = P.masked_attention(q + 50.0, k + 1.0, v, m, 1.0, softcap=3.0, sink=True)   # scores of 100 capped at 3
    want = [n * math.exp(3.0) / (1 + n * math.exp(3.0)) for n in (1, 2, 3, 4, 1, 2, 3, 4, 1, 2)]
    assert torch.allclose(big[:, 0, 0], torch.tensor(want, dtype=torch.float64), rtol=1e-9)
