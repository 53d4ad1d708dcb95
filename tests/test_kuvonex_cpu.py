"""Kuvonex without a GPU: the configuration reader, what the model asks of the loader and of the
cache manager, and identities of the plain implementation that the engine's form rests on."""
import copy

import pytest
import torch

import plain_kuvonex as P
from tiny_kuvonex import CONFIGS, config

from sharpinference_amd import ConfigError, build_model, load_config
from sharpinference_amd.cache.manager import CacheManager
from sharpinference_amd.parts.model import Run


def test_the_architecture_is_found_by_its_one_string_and_round_trips():
    for name in CONFIGS:
        cfg = load_config(config(name))
        assert cfg.architecture == "Kuvonex"
        assert load_config(cfg.to_dict()).to_dict() == cfg.to_dict()
        assert cfg.to_dict()["layers"] == CONFIGS[name]["layers"]


@pytest.mark.parametrize("edit, word", [
    (lambda c: c["layers"][0]["mixer"].update(window=4), "window"),
    (lambda c: c.update(tie=True), "tie"),
    (lambda c: c["layers"][0].update(type="recurrent"), "recurrent"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "dense"),
    (lambda c: c["layers"][1]["mixer"].update(kv_from=2), "earlier"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=1), "latent of its own"),
    (lambda c: c["layers"][1]["mixer"].update(kv_rank=24), "equal"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=4), "divide"),
    (lambda c: c["layers"][3]["mlp"]["router"].update(top=5), "exceeds"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=3), "even"),
    (lambda c: c["layers"][0]["mixer"].pop("heads"), "heads"),
])
def test_a_config_that_cannot_be_this_design_is_refused_with_the_key(edit, word):
    c = config("odd")
    edit(c)
    with pytest.raises(ConfigError) as e:
        load_config(c)
    assert word in str(e.value)


def test_tensor_names_and_shapes_follow_the_layers():
    model = build_model(load_config(config("odd")))
    specs = model.param_specs()
    assert specs["embed"].shape == (97, 64) and specs["head"].shape == (97, 64) and specs["final.norm"].shape == (64,)
    assert specs["l0.mix.q"].shape == (3 * 32, 64) and specs["l0.mix.dkv"].shape == (48, 64)
    assert specs["l0.mix.dkv.norm"].shape == (40,) and specs["l0.mix.uk"].shape == (72, 40)
    assert specs["l0.mix.uv"].shape == (60, 40) and specs["l0.mix.sink"].shape == (3,)
    assert specs["l0.mix.g"].shape == (60, 64) and specs["l0.mix.o"].shape == (64, 60)
    assert "l1.mix.dkv" not in specs and "l1.mix.dkv.norm" not in specs and "l1.mix.uk" in specs
    assert not any(n.startswith("l1.mlp") or n == "l1.norm2" for n in specs) and "l1.norm1" in specs
    assert specs["l3.mlp.e7.down"].shape == (64, 16) and specs["l3.mlp.e0.gate"].shape == (16, 64)
    assert specs["l3.mlp.router"].shape == (8, 64) and specs["l3.mlp.correction"].shape == (8,)
    assert "l3.mlp.e8.up" not in specs


def test_shared_latents_are_one_cache_slot_and_keep_no_value_tensor():
    model = build_model(load_config(config("odd")))
    assert model.schedule == [Run(0, 0), Run(1, 0, write=False), Run(2, 2), Run(3, 2, write=False)]
    specs = model.cache_specs()
    assert specs[1] is None and specs[0].head_dim == 48 and specs[2].head_dim == 48 and specs[0].values_in_keys
    assert specs[0].elements_per_token == 48
    cm = CacheManager(specs, 16, 8, 2, torch.float32, "cpu")
    assert cm.k[0].shape == (8, 1, 16, 48) and cm.v[0] is None and cm.k[1] is None
    assert cm.bytes_per_page() == [2 * 48 * 16 * 4]


# ---------------------------------------------------------------------------
# the plain implementation
# ---------------------------------------------------------------------------
def _weights(name, seed=0, std=0.2):
    model = build_model(load_config(config(name)))
    g = torch.Generator().manual_seed(seed)
    w = {}
    for n, spec in model.param_specs().items():
        if spec.init == "norm_weight":
            w[n] = 0.9 + 0.2 * torch.rand(spec.shape, generator=g, dtype=torch.float64)
        else:
            w[n] = torch.randn(spec.shape, generator=g, dtype=torch.float64) * (1.0 if n.endswith("sink") else std)
    return w


def test_scores_through_the_latent_equal_scores_through_expanded_keys():
    """(q_n^T W_uk) c = q_n . (W_uk c), and W_uv applied to the weighted sum of latents is the
    weighted sum of values: the form the engine computes in is the plain one."""
    c = config("odd")
    w = _weights("odd")
    mx = c["layers"][0]["mixer"]
    H, dn, dr, dv, R = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
    T = 9
    g = torch.Generator().manual_seed(3)
    h = torch.randn(T, c["width"], generator=g, dtype=torch.float64)
    pos = torch.arange(T)
    want, (lat, kr) = P.latent_attention(h, w, "l0.mix.", mx, 1e-5, pos)
    q = (h @ w["l0.mix.q"].T).reshape(T, H, dn + dr)
    q_lat = torch.einsum("thd,hdr->thr", q[..., :dn], w["l0.mix.uk"].reshape(H, dn, R))
    qr = P.rotate(q[..., dn:], pos, mx["rot"]["base"], mx["rot"]["dims"])
    s = (torch.einsum("thr,sr->hts", q_lat, lat) + torch.einsum("thd,sd->hts", qr, kr)) * mx["scale"]
    s = s.masked_fill(pos[None, None, :] > pos[None, :, None], float("-inf"))
    e = torch.exp(s)
    p = e / (e.sum(-1, keepdim=True) + torch.exp(w["l0.mix.sink"])[:, None, None])
    o_lat = torch.einsum("hts,sr->thr", p, lat)
    o = torch.einsum("thr,hvr->thv", o_lat, w["l0.mix.uv"].reshape(H, dv, R)).reshape(T, H * dv)
    got = (o * torch.sigmoid(h @ w["l0.mix.g"].T)) @ w["l0.mix.o"].T
    assert torch.allclose(got, want, atol=1e-10)


def test_a_sink_takes_weight_and_gives_nothing():
    T, H = 4, 2
    g = torch.Generator().manual_seed(1)
    qn, kn, v = (torch.randn(T, H, 5, generator=g, dtype=torch.float64) for _ in range(3))
    qr, kr = torch.randn(T, H, 4, generator=g, dtype=torch.float64), torch.randn(T, 4, generator=g, dtype=torch.float64)
    pos = torch.arange(T)
    off = P.sink_attention(qn, qr, kn, kr, v, torch.full((H,), -1e9, dtype=torch.float64), 0.3, pos, pos)
    on = P.sink_attention(qn, qr, kn, kr, v, torch.tensor([0.0, 50.0], dtype=torch.float64), 0.3, pos, pos)
    assert torch.allclose(off[0], v[0])                       # the first token sees itself alone
    assert on[0, 0].abs().max() < v[0, 0].abs().max()          # one term more in the denominator: less than the value
    assert on[:, 1].abs().max() < 1e-12                        # a huge sink takes all the weight


def test_rotation_turns_pairs_and_leaves_the_rest():
    v = torch.arange(12, dtype=torch.float64).reshape(1, 1, 12) + 1
    out = P.rotate(v.repeat(3, 1, 1), torch.tensor([0, 1, 7]), 100.0, 4)
    assert torch.equal(out[0], v[0]) and torch.equal(out[:, :, 4:], v.repeat(3, 1, 1)[:, :, 4:])
    import math
    a = 7 * 100.0 ** (-2.0 / 4)
    assert abs(float(out[2, 0, 2]) - (3 * math.cos(a) - 4 * math.sin(a))) < 1e-12
    assert abs(float(out[2, 0, 3]) - (4 * math.cos(a) + 3 * math.sin(a))) < 1e-12


def test_experts_are_chosen_with_the_correction_inside_the_best_groups_and_weighted_without_it():
    router = {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 1}}
    wr = torch.eye(6, dtype=torch.float64)
    # scores s = sigmoid(h); group 1 = experts (2, 3) has the best pair sum although expert 0 is the best single one
    h = torch.tensor([[3.0, -3.0, 1.0, 1.2, -1.0, 0.5]], dtype=torch.float64)
    ids, wts = P.route(h, wr, torch.zeros(6, dtype=torch.float64), router)
    assert ids.tolist() == [[3, 2]]
    assert torch.allclose(wts, torch.sigmoid(h[0, [3, 2]])[None], atol=1e-6)
    # a negative correction can make every choice score negative: the other groups still count as minus infinity
    corr = torch.tensor([-5.0, -5.0, -2.0, -2.5, -9.0, -9.0], dtype=torch.float64)
    ids, wts = P.route(h, wr, corr, router)
    assert ids.tolist() == [[2, 3]]
    assert torch.allclose(wts, torch.sigmoid(h[0, [2, 3]])[None], atol=1e-6)     # the weights do not see the correction
    # keep every group: the plain top picks by corrected score
    ids, _ = P.route(h, wr, torch.tensor([0.0, 2.0, 0, 0, 0, 0], dtype=torch.float64), {"experts": 6, "top": 2})
    assert ids.tolist() == [[1, 0]]


def test_the_feed_forward_is_the_weighted_sum_of_the_chosen_experts():
    c = config("odd")
    w = _weights("odd")
    g = torch.Generator().manual_seed(5)
    h = torch.randn(3, c["width"], generator=g, dtype=torch.float64)
    mlp = c["layers"][3]["mlp"]
    ids, wts = P.route(h, w["l3.mlp.router"], w["l3.mlp.correction"], mlp["router"])
    out = P.moe(h, w, "l3.mlp.", mlp)
    t = 1
    want = sum(wts[t, j] * P.expert(h[t:t + 1], w, f"l3.mlp.e{int(ids[t, j])}.")[0] for j in range(3))
    assert torch.allclose(out[t], want, atol=1e-12)
    per = 8 // 2
    assert len({int(e) // per for e in ids[t]}) == 1            # one group kept: all picks are neighbours


def test_a_prefix_gives_the_logits_of_the_whole():
    c = config("odd")
    w = _weights("odd")
    toks = [5, 9, 96, 0, 33, 33, 7, 61, 2, 18, 40]
    whole, layers = P.forward(c, w, toks, want_layers=True)
    part = P.forward(c, w, toks[:6])
    assert torch.allclose(whole[:6], part, atol=1e-9) and layers.shape == (4, len(toks), 64)


def test_the_benchmark_shapes_are_valid_configurations_of_both_architectures():
    import importlib.util
    import os

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("bench_for_test", os.path.join(root, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    for z in bench.KUVONEX_SIZES.values():
        k = load_config(bench.kuvonex_config(z))
        l = load_config(bench.llama4_config_like(z))
        assert k.width == l.hidden_size == z["width"] and len(k.layers) == l.num_hidden_layers == z["layers"]
        assert k.layers[0].mlp.experts == l.num_local_experts and k.layers[0].mlp.ff == l.intermediate_size
        assert k.layers[-1].mixer.kv_from == z["layers"] - 2 and k.layers[0].mixer.kv_from is None
        build_model(k), build_model(l)
