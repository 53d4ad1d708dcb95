"""Kuvonex on the GPU against the plain implementation (tests/plain_kuvonex.py): every mechanism
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

import plain_kuvonex as P
from tiny_kuvonex import CONFIGS, SEEDS, STD_BY_SUFFIX, config

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def _rel_rms(got: torch.Tensor, want: torch.Tensor) -> float:
    """The largest error of a row, as rms(difference) / rms(row)."""
    got, want = got.double().cpu(), want.double().cpu()
    return float(((got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-30)).max())


def _rel_rows(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    got, want = got.double().cpu(), want.double().cpu()
    return (got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-30)


def _bf16_tol(n_layers: int) -> float:
    """rms error of a row of bfloat16 logits relative to the row's rms: every stored tensor is rounded
    to 8 bits (rms 2^-8 / sqrt(12) of its size), thirteen stores a layer add in quadrature, each
    taken to reach the logits with a weight of at most 3 (stated, not derived: the tests' sinks and
    score scales make sharp softmaxes).  Nine rows in ten must lie inside this bound and none
    beyond two and a half times it: single rows are sensitive (one of 150 reaches 0.049 with five
    layers where the ninth decile is 0.020, in the float kernel's and the matrix-core kernel's
    runs alike), while a wrong key, sink, gate or expert puts most rows at 0.05 to 1.  The float32
    runs of the same tests are the sharp ones."""
    return 3.0 * 2.0 ** -8 / math.sqrt(12.0) * math.sqrt(13 * n_layers + 1)


def _tol(dtype: str, n_layers: int = 1) -> float:
    return 2e-5 if dtype == "float32" else _bf16_tol(n_layers)


# ---------------------------------------------------------------------------
# the mechanisms alone
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T, H", [(1, 64), (7, 72), (70, 200)])
def test_norm_on_a_branch_output_is_added_to_the_stream(dtype, T, H):
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(T)
    h = torch.randn(T, H, generator=g)
    y = (torch.randn(T, H, generator=g) * 3).to(DT[dtype])
    w = 0.5 + torch.rand(H, generator=g)
    hd = h.to(DEV)
    act = ops.norm_add(hd, y.to(DEV), w.to(DEV), 1e-5, DT[dtype] if dtype == "bfloat16" else None)
    want = h.double() + P.rms_norm(y.double(), w.double(), 1e-5)
    assert _rel_rms(hd, want) < 1e-6
    if dtype == "bfloat16":
        assert act.dtype == torch.bfloat16 and torch.equal(act.cpu(), hd.cpu().to(torch.bfloat16))
    else:
        assert act is None


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_norm_forms_a_weighted_sum_of_expert_rows_itself(dtype):
    from sharpinference_amd import ops

    T, H, k = 9, 48, 3
    g = torch.Generator().manual_seed(2)
    rows = torch.randn(T * k, H, generator=g).to(DT[dtype])
    perm = torch.randperm(T * k, generator=g).to(torch.int32)
    wts = torch.rand(T, k, generator=g)
    h = torch.randn(T, H, generator=g)
    w = torch.ones(H)
    hd = h.to(DEV)
    lazy = ops.ExpertSum(rows.to(DEV), perm.to(DEV), None, T, k, wts.to(DEV))
    ops.norm_add(hd, lazy, w.to(DEV), 1e-6, None)
    summed = (rows.double()[perm.long()].reshape(T, k, H) * wts.double()[..., None]).sum(1).to(DT[dtype]).double()
    want = h.double() + P.rms_norm(summed, w.double(), 1e-6)
    assert _rel_rms(hd, want) < (1e-6 if dtype == "float32" else 3e-3)
    hd2 = h.to(DEV)
    ops.norm_add(hd2, lazy.tensor(), w.to(DEV), 1e-6, None)          # the combine kernel first: the same row
    assert _rel_rms(hd, hd2.cpu()) < 1e-6


@pytest.mark.parametrize("E, groups, keep, top", [(6, 3, 2, 2), (8, 2, 1, 3), (12, 12, 5, 4), (16, 4, 4, 6), (5, 1, 1, 1),
                                                 (64, 8, 3, 6), (3, 3, 1, 1)])
@pytest.mark.parametrize("T", [1, 7, 70])
def test_router_picks_by_corrected_scores_inside_the_best_groups(E, groups, keep, top, T):
    from sharpinference_amd import ops

    H = 40
    g = torch.Generator().manual_seed(E * 100 + T)
    x = torch.randn(T, H, generator=g)
    wr = torch.randn(E, H, generator=g) * 0.3
    corr = torch.randn(E, generator=g) * 0.7 - 2.0          # choice scores are mostly negative
    ids, wts = ops.router_topk(x.to(DEV), wr.to(DEV), top, ops.GATE_SIGMOID, False, correction=corr.to(DEV),
                               n_groups=groups, keep_groups=keep)
    router = {"experts": E, "top": top, "groups": {"count": groups, "keep": keep}}
    want_ids, want_w = P.route(x.double(), wr.double(), corr.double(), router)
    assert torch.equal(ids.cpu().long(), want_ids), "picks differ"
    assert torch.allclose(wts.cpu().double(), want_w, atol=1e-6)      # the weights carry no correction
    # without a correction and with every group kept the kernel is the plain top-k
    ids0, _ = ops.router_topk(x.to(DEV), wr.to(DEV), top, ops.GATE_SIGMOID, False)
    assert torch.equal(ids0.cpu().long(), torch.sigmoid(x.double() @ wr.double().T).topk(top).indices)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, dn, dr, R, dims", [(3, 24, 8, 40, 8), (4, 16, 16, 32, 6), (2, 8, 32, 64, 32)])
def test_latent_rows_and_rotated_query_parts(dtype, H, dn, dr, R, dims):
    from sharpinference_amd import ops

    T, ps, pages, eps = 11, 16, 5, 1e-5
    g = torch.Generator().manual_seed(H)
    D = R + dr
    proj = torch.randn(T, H * (dn + dr) + 7 + D, generator=g).to(DT[dtype])     # 7 columns that belong to nobody
    kv_off = H * (dn + dr) + 7
    pos = torch.tensor([0, 1, 2, 15, 16, 17, 100, 1000, 31, 32, 5], dtype=torch.int32)
    slots = torch.tensor([3, 17, 40, -1, 79, 0, 5, 6, 7, 8, 9], dtype=torch.int32)
    nw = 0.5 + torch.rand(R, generator=g)
    base = 500.0
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64).float()
    rows = torch.full((pages, 1, ps, D), 7.0).to(DT[dtype]).to(DEV)
    q_full = torch.zeros(T, H * D, dtype=DT[dtype], device=DEV)
    ops.latent_prep(proj.to(DEV), 0, kv_off, q_full, rows, slots.to(DEV), pos.to(DEV), freq.to(DEV), nw.to(DEV), eps,
                    H, dn, dr, R)
    pd = proj.double()
    c = P.rms_norm(pd[:, kv_off:kv_off + R], nw.double(), eps)
    kr = P.rotate(pd[:, kv_off + R:kv_off + D], pos.long(), base, dims)
    qr = P.rotate(pd[:, :H * (dn + dr)].reshape(T, H, dn + dr)[..., dn:], pos.long(), base, dims)
    tol = 5e-5 if dtype == "float32" else 6e-3        # (an angle of 1,000 radians in 32 bits is good to 6e-5)
    flat = rows.cpu().double().reshape(pages * ps, D)
    for t in range(T):
        if slots[t] < 0:
            continue
        assert _rel_rms(flat[slots[t]][None], torch.cat([c[t], kr[t]])[None]) < tol, f"token {t}"
    untouched = torch.ones(pages * ps, dtype=torch.bool)
    untouched[slots[slots >= 0].long()] = False
    assert bool((flat[untouched] == 7.0).all())                  # a slot of -1 stores nothing, nothing else is written
    got_qr = q_full.cpu().double().reshape(T, H, D)[..., R:]
    assert _rel_rms(got_qr.reshape(T, -1), qr.reshape(T, -1)) < tol
    # a layer that makes no latent of its own only rotates its queries
    q2 = torch.zeros_like(q_full)
    ops.latent_prep(proj.to(DEV), 0, None, q2, None, None, pos.to(DEV), freq.to(DEV), None, eps, H, dn, dr, R)
    assert torch.equal(q2.cpu().reshape(T, H, D)[..., R:], q_full.cpu().reshape(T, H, D)[..., R:])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("xo, oo, pad", [(5, 2, 3), (8, 4, 4)])     # unaligned: the float kernel; aligned: the matrix cores in bfloat16
@pytest.mark.parametrize("T, H, N, K", [(1, 3, 40, 24), (70, 5, 12, 40), (130, 2, 64, 64), (33, 4, 100, 136), (17, 1, 4, 8)])
def test_products_per_head_and_the_gate(dtype, T, H, N, K, xo, oo, pad):
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(T)
    sx, so = K + 8, N + pad + 1 if pad == 3 else N + pad
    x = torch.randn(T, xo + H * sx + (3 if pad == 3 else 0), generator=g).to(DT[dtype])
    w = (torch.randn(H, N, K, generator=g) * 0.3).to(DT[dtype])
    gate = torch.randn(T, 9 + H * N, generator=g).to(DT[dtype])
    out = torch.zeros(T, oo + H * so + (1 if pad == 3 else 0), dtype=DT[dtype], device=DEV)
    ops.head_gemm(x.to(DEV), xo, sx, w.to(DEV), out, oo, so, gate=gate.to(DEV), gate_off=9)
    xs = torch.stack([x.double()[:, xo + h * sx: xo + h * sx + K] for h in range(H)], 1)          # [T, H, K]
    want = torch.einsum("thk,hnk->thn", xs, w.double()) * torch.sigmoid(gate.double()[:, 9:].reshape(T, H, N))
    got = torch.stack([out.cpu().double()[:, oo + h * so: oo + h * so + N] for h in range(H)], 1)
    assert _rel_rms(got.reshape(T, -1), want.reshape(T, -1)) < (1e-6 if dtype == "float32" else 4e-3)
    untouched = torch.ones(out.shape[1], dtype=torch.bool)
    for h in range(H):
        untouched[oo + h * so: oo + h * so + N] = False
    assert bool((out.cpu()[:, untouched] == 0).all())                 # nothing is written between the heads' outputs
    plain = torch.zeros_like(out)
    ops.head_gemm(x.to(DEV), xo, sx, w.to(DEV), plain, oo, so)
    got = torch.stack([plain.cpu().double()[:, oo + h * so: oo + h * so + N] for h in range(H)], 1)
    assert _rel_rms(got.reshape(T, -1), torch.einsum("thk,hnk->thn", xs, w.double()).reshape(T, -1)) < (1e-6 if dtype == "float32" else 4e-3)


class _Ctx:
    """What the attention op reads of a step: per-token arrays and the work lists (tokens of one
    request: `tiles` cuts them into prompt tiles of tile_tokens, `singles` lists them one by one)."""

    def __init__(self, entry_of, positions, tiles=False, singles=False, tile_tokens=64):
        self.entry_of_token, self.positions = entry_of, positions
        self.n_decode, self.decode_tokens, self.n_prefill_tiles, self.prefill_tiles = 0, None, 0, None
        self.prefill_tile_tokens = tile_tokens
        T = positions.shape[0]
        if tiles:
            t = [(0, o, min(tile_tokens, T - o)) for o in range(0, T, tile_tokens)]
            self.prefill_tiles = torch.tensor(t, dtype=torch.int32, device=positions.device)
            self.n_prefill_tiles = len(t)
        if singles:
            self.n_decode = T


class _Group:
    def __init__(self, bt, max_context=0):
        self.block_table = bt
        self.max_context = max_context


def _latent_case(H, R, dr, S, dtype, seed, far_key=None, sharpen=30.0):
    """S cached rows of one request on shuffled pages; every position queries.  With far_key, the
    query of the last position and the key at far_key are scaled so that this one score stands out."""
    g = torch.Generator().manual_seed(seed)
    ps, D = 16, R + dr
    n_blocks = (S + ps - 1) // ps
    pages = n_blocks + 3
    perm = torch.randperm(pages, generator=g)[:n_blocks]
    keys = torch.randn(S, D, generator=g)
    q = torch.randn(S, H, D, generator=g)
    if far_key is not None:
        keys[far_key] *= 3.0
        q[S - 1] = keys[far_key][None, :] * (sharpen / keys[far_key].pow(2).sum()) + 0.05 * q[S - 1]
    keys, q = keys.to(DT[dtype]), q.to(DT[dtype])
    rows = torch.zeros(pages, 1, ps, D, dtype=DT[dtype])
    for p in range(S):
        rows[perm[p // ps], 0, p % ps] = keys[p]
    bt = torch.full((1, n_blocks + 2), -1, dtype=torch.int32)
    bt[0, :n_blocks] = perm.to(torch.int32)
    return q, keys, rows, bt


def _plain_latent(q, keys, sink, scale, R, positions):
    """Attention over rows in the plain implementation's terms: one 'head-shared' key per row whose
    first R elements are also the value."""
    qd, kd = q.double(), keys.double()
    H = q.shape[1]
    S = keys.shape[0]
    kn = kd[:, None, :R].expand(S, H, R)
    return P.sink_attention(qd[..., :R], qd[..., R:], kn, kd[:, R:], kn, sink.double(), scale, positions, torch.arange(S))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, R, dr, S", [(3, 40, 8, 50), (5, 64, 16, 130), (4, 96, 32, 33), (1, 8, 2, 17), (9, 300, 20, 70)])
def test_attention_over_latent_rows_with_a_sink(dtype, H, R, dr, S):
    from sharpinference_amd import ops

    q, keys, rows, bt = _latent_case(H, R, dr, S, dtype, seed=S)
    sink = torch.linspace(-6.0, 6.0, H) if H > 1 else torch.tensor([2.0])      # from negligible to dominant
    pos = torch.arange(S, dtype=torch.int32)
    ctx = _Ctx(torch.zeros(S, dtype=torch.int32, device=DEV), pos.to(DEV))
    scale = 1.0 / math.sqrt(R + dr)
    out = ops.attention_latent(q.reshape(S, -1).to(DEV), rows.to(DEV), _Group(bt.to(DEV)), ctx, scale, H, R, dr,
                               sink=sink.to(DEV), kernel="generic")
    want = _plain_latent(q, keys, sink, scale, R, pos.long())
    assert _rel_rms(out.cpu().reshape(S, -1), want.reshape(S, -1)) < (2e-5 if dtype == "float32" else 8e-3)
    none = ops.attention_latent(q.reshape(S, -1).to(DEV), rows.to(DEV), _Group(bt.to(DEV)), ctx, scale, H, R, dr, kernel="generic")
    want0 = _plain_latent(q, keys, torch.full((H,), -1e30), scale, R, pos.long())
    assert _rel_rms(none.cpu().reshape(S, -1), want0.reshape(S, -1)) < (2e-5 if dtype == "float32" else 8e-3)
    assert _rel_rms(out.cpu().reshape(S, -1), want0.reshape(S, -1)) > 0.05      # the sink is no small thing here


@pytest.mark.parametrize("how", ["tiles", "singles"])
@pytest.mark.parametrize("H, R, dr, S", [(3, 64, 16, 50), (5, 96, 16, 130), (8, 96, 16, 1100), (16, 128, 32, 77), (1, 16, 8, 40),
                                         (20, 512, 64, 70), (40, 256, 32, 300), (70, 32, 0, 65), (6, 80, 24, 150), (2, 80, 24, 150),
                                         (4, 48, 8, 150), (12, 48, 8, 150), (24, 208, 8, 90), (7, 400, 40, 45)])
def test_the_matrix_core_kernel_over_latent_rows(H, R, dr, S, how):
    """Prompt tiles and listed single tokens through the matrix-core kernel: rows of several tokens in a
    wave (few heads), several head tiles (many heads), one run and several (merged afterwards)."""
    from sharpinference_amd import ops

    q, keys, rows, bt = _latent_case(H, R, dr, S, "bfloat16", seed=S + H)
    sink = torch.linspace(-4.0, 4.0, H) if H > 1 else torch.tensor([1.0])
    pos = torch.arange(S, dtype=torch.int32)
    scale = 1.0 / math.sqrt(R + dr)
    want = _plain_latent(q, keys, sink, scale, R, pos.long())
    ctx = _Ctx(torch.zeros(S, dtype=torch.int32, device=DEV), pos.to(DEV), tiles=how == "tiles", singles=how == "singles")
    assert ops.latent_mfma_ok(torch.bfloat16, R, dr)
    out = ops.attention_latent(q.reshape(S, -1).to(DEV), rows.to(DEV), _Group(bt.to(DEV), S), ctx, scale, H, R, dr,
                               sink=sink.to(DEV), kernel="mfma")
    assert _rel_rms(out.cpu().reshape(S, -1), want.reshape(S, -1)) < 8e-3
    # the same rows through the float kernel, and without sinks
    gen = ops.attention_latent(q.reshape(S, -1).to(DEV), rows.to(DEV), _Group(bt.to(DEV), S), ctx, scale, H, R, dr,
                               sink=sink.to(DEV), kernel="generic")
    assert _rel_rms(out.cpu().reshape(S, -1), gen.cpu().reshape(S, -1)) < 8e-3
    none = ops.attention_latent(q.reshape(S, -1).to(DEV), rows.to(DEV), _Group(bt.to(DEV), S), ctx, scale, H, R, dr, kernel="mfma")
    want0 = _plain_latent(q, keys, torch.full((H,), -1e30), scale, R, pos.long())
    assert _rel_rms(none.cpu().reshape(S, -1), want0.reshape(S, -1)) < 8e-3


def test_sizes_the_matrix_core_kernel_refuses_go_to_the_float_kernel():
    from sharpinference_amd import ops

    assert not ops.latent_mfma_ok(torch.bfloat16, 40, 8) and not ops.latent_mfma_ok(torch.float32, 64, 16)
    assert not ops.latent_mfma_ok(torch.bfloat16, 64, 12) and not ops.latent_mfma_ok(torch.bfloat16, 512, 192)
    assert ops.latent_run_keys(700, False) == ops.latent_run_keys(70000, False) == ops.LATENT_DECODE_RUN_KEYS
    assert [ops.latent_run_keys(n, True) for n in (5, 2048, 2049, 9000)] == [1024, 1024, 2048, 8192]


@pytest.mark.parametrize("far_key", [0, 15, 16, 17, 1023, 1024, 1025, 1097])
def test_one_key_among_a_thousand_is_found_in_a_prompt_tile(far_key):
    """The same through prompt tiles of the matrix-core kernel: 1,099 positions query at once, the
    last one looks for the key; keys on both sides of the 1,024-key run border and of page borders."""
    from sharpinference_amd import ops

    H, R, dr, S = 4, 64, 16, 1099
    q, keys, rows, bt = _latent_case(H, R, dr, S, "bfloat16", seed=far_key, far_key=far_key)
    sink = torch.zeros(H)
    pos = torch.arange(S, dtype=torch.int32)
    ctx = _Ctx(torch.zeros(S, dtype=torch.int32, device=DEV), pos.to(DEV), tiles=True)
    out = ops.attention_latent(q.reshape(S, -1).to(DEV), rows.to(DEV), _Group(bt.to(DEV), S), ctx, 1.0, H, R, dr,
                               sink=sink.to(DEV), kernel="mfma")
    want = _plain_latent(q[S - 1:], keys, sink, 1.0, R, pos[S - 1:].long())
    assert _rel_rms(want.reshape(1, -1), keys[far_key, :R].double().repeat(H)[None]) < 0.05
    assert _rel_rms(out.cpu()[S - 1:].reshape(1, -1), want.reshape(1, -1)) < 1e-2


@pytest.mark.parametrize("dtype, kernel", [("float32", "generic"), ("bfloat16", "generic"), ("bfloat16", "mfma")])
@pytest.mark.parametrize("far_key", [0, 3, 15, 16, 17, 127, 128, 129, 255, 256, 640, 689])
def test_one_key_among_hundreds_is_found_wherever_it_lies(dtype, kernel, far_key):
    from sharpinference_amd import ops

    H, R, dr, S = 4, 64, 16, 691
    q, keys, rows, bt = _latent_case(H, R, dr, S, dtype, seed=far_key, far_key=far_key)
    sink = torch.zeros(H)
    last = torch.tensor([S - 1], dtype=torch.int32)
    ctx = _Ctx(torch.zeros(1, dtype=torch.int32, device=DEV), last.to(DEV), singles=True)
    out = ops.attention_latent(q[S - 1:].reshape(1, -1).to(DEV), rows.to(DEV), _Group(bt.to(DEV), S), ctx, 1.0, H, R, dr,
                               sink=sink.to(DEV), kernel=kernel)
    want = _plain_latent(q[S - 1:], keys, sink, 1.0, R, last.long())
    # the key that stands out carries the result: leaving it out (or taking its neighbour) is an error of order one
    assert _rel_rms(want.reshape(1, -1), keys[far_key, :R].double().repeat(H)[None]) < 0.05
    assert _rel_rms(out.cpu().reshape(1, -1), want.reshape(1, -1)) < (2e-5 if dtype == "float32" else 1e-2)


# ---------------------------------------------------------------------------
# the engine
# ---------------------------------------------------------------------------
@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    from sharpinference_amd import load_config
    from sharpinference_amd.weights.loader import write_random_model

    out = {}
    for name in CONFIGS:
        d = str(tmp_path_factory.mktemp("kuvonex_" + name))
        write_random_model(load_config(config(name)), d, SEEDS[name], std=0.1, std_by_suffix=STD_BY_SUFFIX)
        out[name] = d
    return out


@functools.lru_cache(maxsize=4)
def _plain_model(d):
    return P.read_config(d), P.load_weights(d, torch.float64)


def _moe_layers(cfg):
    return [i for i, l in enumerate(cfg["layers"]) if l.get("mlp") is not None]


def _engine(d, dtype, **kw):
    from sharpinference_amd.engine import Engine

    args = dict(dtype=dtype, device=DEV, max_num_seqs=4, kv_tokens=1024, max_model_len=1024)
    args.update(kw)
    return Engine(d, **args)


def _run(eng, reqs, steps, free=True):
    """steps: lists of (request id, number of its next tokens).  Returns per request the logits at
    every position [T, V] and, per routed layer, the experts the engine picked [T, top]."""
    from sharpinference_amd.engine import StepEntry

    at = {r: 0 for r in reqs}
    logits = {r: [] for r in reqs}
    picks = {r: None for r in reqs}
    for step in steps:
        entries = []
        for r, n in step:
            if at[r] == 0:
                eng.add_request(r)
            entries.append(StepEntry(r, reqs[r][at[r]:at[r] + n], list(range(n))))
        trace = []
        out = eng.step(entries, router_trace=trace).cpu()
        o = 0
        for r, n in step:
            logits[r].append(out[o:o + n])
            if picks[r] is None:
                picks[r] = [[] for _ in trace]
            for li, item in enumerate(trace):
                picks[r][li].append(item[0][o:o + n].cpu().long())
            o += n
            at[r] += n
            if at[r] == len(reqs[r]) and free:
                eng.free_request(r)
    return ({r: torch.cat(v) for r, v in logits.items()},
            {r: [torch.cat(p) for p in v] for r, v in picks.items()})


def _check(d, dtype, reqs, got, picks, what):
    cfg, w = _plain_model(d)
    layers = _moe_layers(cfg)
    for r, toks in reqs.items():
        use = dict(zip(layers, picks[r])) if dtype == "bfloat16" else None     # float32 must pick as the plain one does
        want = P.forward(cfg, w, toks, picks=use)
        err = _rel_rows(got[r], want)
        if dtype == "float32":
            assert float(err.max()) < 5 * _tol(dtype), f"{what}, request {r}: {float(err.max()):.2e}"
            continue
        tol = _tol(dtype, len(cfg["layers"]))
        ninth = float(torch.quantile(err, 0.9)) if err.numel() > 1 else float(err.max())
        assert ninth < tol and float(err.max()) < 2.5 * tol, \
            f"{what}, request {r}: ninth decile {ninth:.2e}, worst {float(err.max()):.2e} (bound {tol:.2e})"


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
@pytest.mark.parametrize("name", ["odd", "even", "mid"])
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
        got, picks = _run(eng, {what: toks}, [[(what, n)] for n in cuts])
        _check(d, dtype, {what: toks}, got, picks, f"{name} {dtype} {what}")
        if dtype == "float32":
            first = got[what] if first is None else first
            assert _rel_rms(got[what], first) < 1e-5, f"{what}: the cut changes the logits"
    if dtype == "bfloat16":
        assert eng.runner.graph_replays > 0                       # decode steps ran from graphs
    eng.cache.check_invariants()
    assert not eng.cache.requests


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_requests_in_one_batch_give_what_each_gives_alone(model_dirs, dtype):
    d = model_dirs["odd"]
    vocab = CONFIGS["odd"]["vocab"]
    reqs = {"a": _tokens(90, vocab, 2), "b": _tokens(37, vocab, 3), "c": _tokens(130, vocab, 4), "d": _tokens(5, vocab, 5)}
    steps = [[("a", 29), ("b", 2)], [("a", 1), ("b", 33), ("c", 64)], [("c", 2), ("a", 1), ("d", 5), ("b", 1)],
             [("a", 59), ("c", 1), ("b", 1)], [("c", 63)]]
    eng = _engine(d, dtype)
    got, picks = _run(eng, reqs, steps)
    _check(d, dtype, reqs, got, picks, f"mixed {dtype}")
    if dtype == "float32":
        for r, toks in reqs.items():
            alone, _ = _run(eng, {r: toks}, [[(r, len(toks))]])
            assert _rel_rms(got[r], alone[r]) < 1e-5, f"{r}: the batch changes the logits"
    eng.cache.check_invariants()


def test_pages_and_slots_are_given_back_and_used_again(model_dirs):
    d = model_dirs["even"]
    vocab = CONFIGS["even"]["vocab"]
    eng = _engine(d, "float32", max_num_seqs=2, kv_tokens=192, max_model_len=160)
    pool = eng.cache.groups[0].pool
    assert pool.num_pages == 12
    slots = set()
    for i in range(5):
        a, b = f"a{i}", f"b{i}"
        reqs = {a: _tokens(100 + i, vocab, 10 + i), b: _tokens(60 - i, vocab, 20 + i)}
        steps = [[(a, 40), (b, 3)], [(a, 60 + i), (b, 57 - i - 1)], [(b, 1)]]
        eng.add_request(a), eng.add_request(b)
        slots |= {eng.cache.requests[a].state_slot, eng.cache.requests[b].state_slot}
        eng.free_request(a), eng.free_request(b)
        got, picks = _run(eng, reqs, steps)
        _check(d, "float32", reqs, got, picks, f"round {i}")
        eng.cache.check_invariants()
    assert pool.total_allocs > 3 * pool.num_pages and pool.num_free == pool.num_pages and len(slots) == 2


def test_a_sink_or_a_correction_left_out_would_show(model_dirs):
    """The weights of these tests make both matter: the plain model without them is far from the engine."""
    d = model_dirs["odd"]
    cfg, w = _plain_model(d)
    toks = _tokens(60, CONFIGS["odd"]["vocab"], 6)
    eng = _engine(d, "float32")
    got, _ = _run(eng, {"x": toks}, [[("x", 60)]])
    no_sink = {k: (torch.full_like(v, -1e30) if k.endswith(".sink") else v) for k, v in w.items()}
    assert _rel_rms(got["x"], P.forward(cfg, no_sink, toks)) > 0.02
    no_corr = {k: (torch.zeros_like(v) if k.endswith(".correction") else v) for k, v in w.items()}
    assert _rel_rms(got["x"], P.forward(cfg, no_corr, toks)) > 0.02
    assert _rel_rms(got["x"], P.forward(cfg, w, toks)) < 1e-4


@pytest.mark.parametrize("name", ["odd", "even"])
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
    assert _rel_rms(read(0, 2), wa[[0, 32]]) < 1e-4
    assert _rel_rms(read(1, 1), wb[[19]]) < 1e-4
    assert _rel_rms(read(2, 1), wa[[68]]) < 1e-4 and _rel_rms(read(3, 1), wa[[69]]) < 1e-4
