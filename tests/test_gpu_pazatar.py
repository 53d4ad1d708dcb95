"""Pazatar on the GPU against the plain implementation (tests/plain_pazatar.py): every mechanism
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

import plain_pazatar as P
from tiny_pazatar import CONFIGS, SEEDS, STD_BY_SUFFIX, config, runs_of

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def _rel_rows(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    got, want = got.double().cpu(), want.double().cpu()
    return (got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-30)


def _rel_rms(got: torch.Tensor, want: torch.Tensor) -> float:
    """The largest error of a row, as rms(difference) / rms(row)."""
    return float(_rel_rows(got, want).max())


def _bf16_tol(n_runs: int) -> float:
    """rms error of a row of bfloat16 logits relative to the row's rms: every stored tensor is rounded
    to 8 bits (rms 2^-8 / sqrt(12) of its size), some twenty stores a layer run add in quadrature,
    each taken to reach the logits with a weight of at most 3 (stated, not derived).  Nine rows in
    ten must lie inside this bound, at most three in a hundred beyond two and a half times it, and
    none beyond a half of the row's size: single rows are sensitive (on the second configuration row
    105 of one 130-token request is 0.237 off and row 147 of a 150-token one 0.14, where the ninth
    deciles are 0.017 and 0.024: to four digits the same whether the request runs whole, in
    portions or inside a mixed batch, and the same in the float attention kernel's and the
    matrix-core kernels' runs), while a wrong key, sink, state or chunk edge puts the rows it
    touches at order one.  The float32 runs of the same tests are the sharp ones."""
    return 3.0 * 2.0 ** -8 / math.sqrt(12.0) * math.sqrt(20 * n_runs + 1)


class _Step:
    """What the kernels between projections and attention read of a step."""

    def __init__(self, lens, starts, slots):
        self.n_entries, self.n_tokens, self.max_entry_len = len(lens), sum(lens), max(lens)
        cu = [0]
        for n in lens:
            cu.append(cu[-1] + n)
        self.cu_tokens = torch.tensor(cu, dtype=torch.int32, device=DEV)
        self.entry_of_token = torch.tensor([e for e, n in enumerate(lens) for _ in range(n)], dtype=torch.int32, device=DEV)
        self.positions = torch.tensor([s + i for s, n in zip(starts, lens) for i in range(n)], dtype=torch.int32, device=DEV)
        self.state_slots = torch.tensor(slots, dtype=torch.int32, device=DEV)


# ---------------------------------------------------------------------------
# the mechanisms alone
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, G, d, e, norm, layout, dims, mag, taps, own_v", [
    (3, 3, 10, 10, "projection", "interleaved", 6, 1.3, 0, False),
    (8, 2, 32, 32, "projection", "interleaved", 32, 1.0, 0, False),
    (4, 2, 12, 20, "head", "half", 4, 1.0, 3, True),
    (2, 1, 64, 64, "head", "half", 64, 1.0, 4, True),
    (2, 2, 16, 6, None, "half", 0, 1.0, 2, True),
    (5, 5, 8, 8, "head", "interleaved", 2, 0.7, 8, True),
])
def test_convolution_norm_rotation_and_cache_write(dtype, H, G, d, e, norm, layout, dims, mag, taps, own_v):
    """Two requests in two steps each (the second step of one shorter than the convolution's reach),
    on shuffled pages: q, the cached keys and values and the carried tails against the plain pieces
    applied to the whole sequences."""
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(H * 100 + d + taps)
    ps, eps = 16, 1e-5
    qn, kn, vn = H * d, G * d, (G * e if own_v else 0)
    C, pad = qn + kn + vn, 5                                     # (the projections sit inside a wider row)
    lens = {"a": [19, 1], "b": [2, 30]}
    total = {r: sum(v) for r, v in lens.items()}
    proj = {r: (torch.randn(total[r], C + pad, generator=g) * 2).to(DT[dtype]) for r in lens}
    conv_w = torch.randn(C, taps, generator=g) if taps else None
    wq = 0.5 + torch.rand(qn if norm == "projection" else d, generator=g)
    wk = 0.5 + torch.rand(kn if norm == "projection" else d, generator=g)
    freqs = [1.0 / (3.0 + i) for i in range(dims // 2)]
    # the plain pieces on whole sequences
    want = {}
    for r in lens:
        u = proj[r].double()[:, pad:]
        if taps:
            u = P.short_convolution(u, conv_w.double())
        q, k = u[:, :qn], u[:, qn:qn + kn]
        v = u[:, qn + kn:].reshape(-1, G, e) if own_v else k.reshape(-1, G, d).clone()
        if norm == "projection":
            q, k = P.rms_norm(q, wq.double(), eps), P.rms_norm(k, wk.double(), eps)
        q, k = q.reshape(-1, H, d), k.reshape(-1, G, d)
        if norm == "head":
            q, k = P.rms_norm(q, wq.double(), eps), P.rms_norm(k, wk.double(), eps)
        if dims:
            pos = torch.arange(total[r])
            q, k = P.rotate(q, pos, freqs, layout, mag), P.rotate(k, pos, freqs, layout, mag)
        want[r] = (q, k, v)
    # the kernel, step by step
    pages = 8
    perm = torch.randperm(pages, generator=g).tolist()
    page_of = {"a": perm[:2], "b": perm[2:4]}
    kc = torch.zeros(pages, G, ps, d, dtype=DT[dtype], device=DEV)
    vc = torch.zeros(pages, G, e, ps, dtype=DT[dtype], device=DEV)
    tail = torch.zeros(3, max(taps - 1, 1), C, device=DEV) if taps else None
    slot_of = {"a": 2, "b": 0}
    inv_freq = torch.tensor(freqs, dtype=torch.float32, device=DEV) if dims else None
    mode = {None: ops.NORM_NONE, "head": ops.NORM_PER_HEAD, "projection": ops.NORM_WHOLE}[norm]
    got_q = {r: [] for r in lens}
    at = {r: 0 for r in lens}
    for step in range(2):
        order = ["a", "b"] if step == 0 else ["b", "a"]
        n = [lens[r][step] for r in order]
        ctx = _Step(n, [at[r] for r in order], [slot_of[r] for r in order])
        rows = torch.cat([proj[r][at[r]:at[r] + lens[r][step]] for r in order]).to(DEV)
        slots = torch.tensor([page_of[r][p // ps] * ps + p % ps for r in order for p in range(at[r], at[r] + lens[r][step])],
                             dtype=torch.int32, device=DEV)
        q = ops.qk_prep(rows, pad, pad + qn, pad + qn + kn if own_v else None, H, G, d, e, ctx, kc, vc, slots, mode,
                        wq.to(DEV) if norm else None, wk.to(DEV) if norm else None, eps, inv_freq,
                        ops.PAIRS_HALF_SPLIT if layout == "half" else ops.PAIRS_INTERLEAVED, mag,
                        conv_w.to(DEV) if taps else None, tail)
        o = 0
        for r, m in zip(order, n):
            got_q[r].append(q[o:o + m].cpu())
            o += m
            at[r] += m
    tol = 2e-6 if dtype == "float32" else 6e-3
    for r in lens:
        q, k, v = want[r]
        assert _rel_rms(torch.cat(got_q[r]).reshape(total[r], -1), q.reshape(total[r], -1)) < tol, f"q of {r}"
        got_k = torch.stack([kc[page_of[r][p // ps], :, p % ps].cpu() for p in range(total[r])])
        got_v = torch.stack([vc[page_of[r][p // ps], :, :, p % ps].cpu() for p in range(total[r])])
        assert _rel_rms(got_k.reshape(total[r], -1), k.reshape(total[r], -1)) < tol, f"k of {r}"
        assert _rel_rms(got_v.reshape(total[r], -1), v.reshape(total[r], -1)) < tol, f"v of {r}"
        if taps:      # the tail holds the last taps - 1 projected rows, oldest first
            last = proj[r].float()[-(taps - 1):, pad:pad + C]
            assert torch.equal(tail[slot_of[r], :taps - 1].cpu(), last), f"tail of {r}"
    if taps:
        assert float(tail[1].abs().max()) == 0.0               # a slot no entry named stays untouched


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, dk, dv, tau", [(2, 10, 24, 3.0), (6, 48, 64, 16.0), (1, 136, 20, 0.5), (3, 72, 50, 1.0), (2, 256, 16, 4.0),
                                            (4, 32, 33, 8.0)])
def test_the_recurrence_walks_every_entry_from_its_slots_state(dtype, H, dk, dv, tau):
    """Three requests over five steps (one token, a few, many; a request left out of a step) against
    the plain recurrence over whole sequences; states in slots 3, 0 and 1 of five."""
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(dk + dv)
    qk, vv = H * dk, H * dv
    pad = 3 if dk % 16 else 8                                    # (rows of eight aligned elements take the wide loads)
    plan = [[("a", 1), ("b", 40)], [("b", 1), ("c", 7), ("a", 2)], [("a", 9), ("c", 1)],
            [("c", 1), ("a", 2), ("b", 1)], [("b", 1)]]           # (the last two: single tokens and pairs only, the short-stage form)
    total = {"a": 14, "b": 43, "c": 9}
    slot_of = {"a": 3, "b": 0, "c": 1}
    proj = {r: torch.randn(n, pad + 2 * qk + vv, generator=g).to(DT[dtype]) for r, n in total.items()}
    z = {r: torch.randn(n, qk, generator=g) * 2 for r, n in total.items()}
    bias = torch.randn(qk, generator=g)
    state = torch.zeros(5, *ops.gla_state_shape(H, dk, dv), device=DEV)
    state[2].fill_(9.0)                                          # a slot no entry names
    got = {r: [] for r in total}
    at = {r: 0 for r in total}
    for step in plan:
        ctx = _Step([n for _, n in step], [at[r] for r, _ in step], [slot_of[r] for r, _ in step])
        rows = torch.cat([proj[r][at[r]:at[r] + n] for r, n in step]).to(DEV)
        zz = torch.cat([z[r][at[r]:at[r] + n] for r, n in step]).to(DEV)
        decays = ops.gla_decays(zz, bias.to(DEV), tau)
        assert decays.data_ptr() == zz.data_ptr()              # made in place over the logits
        o = ops.gla_walk(rows, pad, pad + qk, pad + 2 * qk, decays, dk ** -0.5, state, ctx, H, dk, dv)
        i = 0
        for r, n in step:
            got[r].append(o[i:i + n].cpu())
            i += n
            at[r] += n
    for r, n in total.items():
        p = proj[r].double()
        alpha = torch.exp(torch.nn.functional.logsigmoid(z[r].double() + bias.double()) / tau).reshape(n, H, dk)
        want = P.gated_recurrence(p[:, pad:pad + qk].reshape(n, H, dk) * dk ** -0.5, p[:, pad + qk:pad + 2 * qk].reshape(n, H, dk),
                                  p[:, pad + 2 * qk:].reshape(n, H, dv), alpha)
        assert _rel_rms(torch.cat(got[r]), want.reshape(n, -1)) < 2e-6, r      # float arithmetic in both dtypes
    assert float((state[2] - 9.0).abs().max()) == 0.0 and float(state[4].abs().max()) == 0.0
    # what the slots hold in the end are the matrices S of the plain recurrence: sum_s (prod of later decays) k_s v_s^T
    for r, n in total.items():
        p = proj[r].double()
        alpha = torch.exp(torch.nn.functional.logsigmoid(z[r].double() + bias.double()) / tau).reshape(n, H, dk)
        k, v = p[:, pad + qk:pad + 2 * qk].reshape(n, H, dk), p[:, pad + 2 * qk:].reshape(n, H, dv)
        S = torch.zeros(H, dk, dv, dtype=torch.float64)
        for t in range(n):
            S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        got_S = ops.gla_state_matrices(state[slot_of[r]], dk, dv).cpu()
        assert _rel_rms(got_S.reshape(1, -1), S.reshape(1, -1)) < 2e-6, f"state of {r}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, dk, dv, tau", [(2, 48, 64, 16.0), (1, 136, 20, 0.5), (3, 10, 24, 1.0)])
def test_long_entries_walked_in_segments_side_by_side(dtype, H, dk, dv, tau):
    """Two requests, each a long portion after a short one (so that the walk starts from a state that
    is not zero): 700 and 129 tokens in one step, in segments of 128 (a last segment of 60 tokens, one of
    a single token), against the plain recurrence; the states left in the slots against the whole walk's."""
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(dk * 7 + dv)
    qk, vv, pad = H * dk, H * dv, 8
    total = {"a": 705, "b": 132}
    plan = [[("a", 5), ("b", 3)], [("b", 129), ("a", 700)]]
    slot_of = {"a": 1, "b": 0}
    proj = {r: torch.randn(n, pad + 2 * qk + vv, generator=g).to(DT[dtype]) for r, n in total.items()}
    z = {r: torch.randn(n, qk, generator=g) * 2 + 2.0 for r, n in total.items()}
    bias = torch.randn(qk, generator=g)
    states = {}
    outs = {}
    for how in ("whole", "segments"):
        state = torch.zeros(2, *ops.gla_state_shape(H, dk, dv), device=DEV)
        got = {r: [] for r in total}
        at = {r: 0 for r in total}
        for step in plan:
            lens = [n for _, n in step]
            ctx = _Step(lens, [at[r] for r, _ in step], [slot_of[r] for r, _ in step])
            rows = torch.cat([proj[r][at[r]:at[r] + n] for r, n in step]).to(DEV)
            decays = ops.gla_decays(torch.cat([z[r][at[r]:at[r] + n] for r, n in step]).to(DEV), bias.to(DEV), tau)
            segments = None
            if how == "segments" and max(lens) > 128:
                segs, ents = ops.gla_segments(lens, ctx.cu_tokens.cpu().numpy())
                assert segs.shape == (8, 4) and ents.tolist() == [[0, 2], [2, 6]] and segs[1].tolist() == [0, 128, 1, 1]
                segments = (torch.from_numpy(segs).to(DEV), torch.from_numpy(ents).to(DEV))
            o = ops.gla_walk(rows, pad, pad + qk, pad + 2 * qk, decays, dk ** -0.5, state, ctx, H, dk, dv, segments=segments)
            i = 0
            for r, n in step:
                got[r].append(o[i:i + n].cpu())
                i += n
                at[r] += n
        outs[how] = {r: torch.cat(v) for r, v in got.items()}
        states[how] = ops.gla_state_matrices(state, dk, dv).cpu()
    for r, n in total.items():
        p = proj[r].double()
        alpha = torch.exp(torch.nn.functional.logsigmoid(z[r].double() + bias.double()) / tau).reshape(n, H, dk)
        want = P.gated_recurrence(p[:, pad:pad + qk].reshape(n, H, dk) * dk ** -0.5, p[:, pad + qk:pad + 2 * qk].reshape(n, H, dk),
                                  p[:, pad + 2 * qk:].reshape(n, H, dv), alpha)
        assert _rel_rms(outs["segments"][r], want.reshape(n, -1)) < 3e-6, r
        assert _rel_rms(outs["whole"][r], want.reshape(n, -1)) < 3e-6, r
    assert _rel_rms(states["segments"].reshape(2, -1), states["whole"].reshape(2, -1)) < 3e-6


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T, N, rank, tau", [(1, 20, 5, 3.0), (19, 288, 16, 16.0), (70, 520, 64, 0.5), (9, 40, 256, 1.0)])
def test_decays_from_the_narrow_middle_of_their_projection(dtype, T, N, rank, tau):
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(T + rank)
    pad = 11
    proj = torch.randn(T, pad + rank + 2, generator=g).to(DT[dtype])
    w = torch.randn(N, rank, generator=g).to(DT[dtype])
    bias = torch.randn(N, generator=g) * 2
    got = ops.gla_decays_from_middle(proj.to(DEV), pad, rank, w.to(DEV), bias.to(DEV), tau)
    z = proj.double()[:, pad:pad + rank] @ w.double().T + bias.double()
    want = torch.exp(torch.nn.functional.logsigmoid(z) / tau)
    assert got.dtype == torch.float32 and float((got.cpu().double() - want).abs().max()) < 2e-6     # decays lie in (0, 1)
    two = ops.gla_decays((proj[:, pad:pad + rank].float() @ w.float().T).to(DEV), bias.to(DEV), tau)   # the two-kernel form
    assert float((two.cpu().double() - want).abs().max()) < 1e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_head_norm_with_gate_the_join_of_branches_and_the_squared_relu(dtype):
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(5)
    T, H, dv, pad = 9, 3, 20, 7
    o = torch.randn(T, H * dv, generator=g) * 5
    w = 0.5 + torch.rand(dv, generator=g)
    proj = torch.randn(T, pad + H * dv, generator=g).to(DT[dtype])
    y = ops.head_norm_gate(o.to(DEV), w.to(DEV), 1e-5, H, dv, DT[dtype], proj.to(DEV), pad)
    want = (P.rms_norm(o.double().reshape(T, H, dv), w.double(), 1e-5).reshape(T, -1) * P.silu(proj.double()[:, pad:]))
    tol = 2e-6 if dtype == "float32" else 5e-3
    assert _rel_rms(y, want) < tol
    y = ops.head_norm_gate(o.to(DEV), w.to(DEV), 1e-5, H, dv, DT[dtype])
    assert _rel_rms(y, P.rms_norm(o.double().reshape(T, H, dv), w.double(), 1e-5).reshape(T, -1)) < tol
    a, b = (torch.randn(T, 72, generator=g) * 3).to(DT[dtype]), (torch.randn(T, 72, generator=g) * 0.1).to(DT[dtype])
    wa, wb = 0.5 + torch.rand(72, generator=g), 0.5 + torch.rand(72, generator=g)
    j = ops.norm_mean([a.to(DEV), b.to(DEV)], [wa.to(DEV), wb.to(DEV)], 1e-5)
    assert j.dtype == torch.float32
    assert _rel_rms(j, 0.5 * (P.rms_norm(a.double(), wa.double(), 1e-5) + P.rms_norm(b.double(), wb.double(), 1e-5))) < 2e-6
    assert _rel_rms(ops.norm_mean([a.to(DEV)], [wa.to(DEV)], 1e-5), P.rms_norm(a.double(), wa.double(), 1e-5)) < 2e-6
    x = torch.randn(T, 50, generator=g).to(DT[dtype])
    assert _rel_rms(ops.activation(x.to(DEV), "relu2"), P.relu_squared(x.double())) < tol


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T, N", [(1, 72), (9, 320), (70, 2048)])
def test_the_norm_behind_a_branch_and_the_norm_before_the_next_in_one_launch(dtype, T, N):
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(T + N)
    h = torch.randn(T, N, generator=g) * 3
    y = (torch.randn(T, N, generator=g) * 0.2).to(DT[dtype])
    a, b = (torch.randn(T, N, generator=g) * 5).to(DT[dtype]), (torch.randn(T, N, generator=g) * 0.3).to(DT[dtype])
    wp, wn, wa, wb = (0.5 + torch.rand(N, generator=g) for _ in range(4))
    eps = 1e-5
    tol = 2e-6 if dtype == "float32" else 6e-3
    # one branch, with and without the next norm
    hd = h.to(DEV)
    out = ops.post_pre_norm(hd, y.to(DEV), wp.to(DEV), eps, wn.to(DEV), DT[dtype])
    want_h = h.double() + P.rms_norm(y.double(), wp.double(), eps)
    assert _rel_rms(hd, want_h) < 2e-6 and out.dtype == DT[dtype]
    assert _rel_rms(out, P.rms_norm(want_h, wn.double(), eps)) < tol
    hd2 = h.to(DEV)
    assert ops.post_pre_norm(hd2, y.to(DEV), wp.to(DEV), eps) is None and torch.equal(hd2, hd)
    hd3 = h.to(DEV)
    ops.norm_add(hd3, y.to(DEV), wp.to(DEV), eps, None)                       # the unfused kernel: the same sum
    assert _rel_rms(hd3, hd.cpu()) < 1e-6
    # the join of two branches formed on the way
    hd = h.to(DEV)
    join = ops.BranchMean([a.to(DEV), b.to(DEV)], [wa.to(DEV), wb.to(DEV)], eps)
    out = ops.post_pre_norm(hd, join, wp.to(DEV), eps, wn.to(DEV), DT[dtype])
    mean = 0.5 * (P.rms_norm(a.double(), wa.double(), eps) + P.rms_norm(b.double(), wb.double(), eps))
    want_h = h.double() + P.rms_norm(mean, wp.double(), eps)
    assert _rel_rms(join.tensor(), mean) < 2e-6
    assert _rel_rms(hd, want_h) < 2e-6 and _rel_rms(out, P.rms_norm(want_h, wn.double(), eps)) < tol


class _Ctx:
    """What the attention op reads of a step of one request: `tiles` cuts its tokens into prompt
    tiles, `singles` lists them one by one."""

    def __init__(self, positions, tiles=False, singles=False, tile_tokens=64):
        T = positions.shape[0]
        self.entry_of_token, self.positions = torch.zeros(T, dtype=torch.int32, device=DEV), positions.to(DEV)
        self.n_decode, self.decode_tokens, self.n_prefill_tiles, self.prefill_tiles = 0, None, 0, None
        self.prefill_tile_tokens = tile_tokens
        if tiles:
            t = [(0, o, min(tile_tokens, T - o)) for o in range(0, T, tile_tokens)]
            self.prefill_tiles = torch.tensor(t, dtype=torch.int32, device=DEV)
            self.n_prefill_tiles = len(t)
        if singles:
            self.n_decode = T


class _Group:
    def __init__(self, bt, max_context=0):
        self.block_table, self.max_context = bt.to(DEV), max_context


def _paged(k, v, dtype, seed):
    """Keys [S, G, d] and values [S, G, e] of one request on shuffled pages of 16."""
    S, G, d = k.shape
    e = v.shape[2]
    ps = 16
    n_blocks = (S + ps - 1) // ps
    perm = torch.randperm(n_blocks + 3, generator=torch.Generator().manual_seed(seed))[:n_blocks]
    kc = torch.zeros(n_blocks + 3, G, ps, d, dtype=DT[dtype])
    vc = torch.zeros(n_blocks + 3, G, e, ps, dtype=DT[dtype])
    for p in range(S):
        kc[perm[p // ps], :, p % ps] = k[p].to(DT[dtype])
        vc[perm[p // ps], :, :, p % ps] = v[p].to(DT[dtype])
    bt = torch.full((1, n_blocks + 2), -1, dtype=torch.int32)
    bt[0, :n_blocks] = perm.to(torch.int32)
    return kc.to(DEV), vc.to(DEV), bt


def _attention_case(S, H, G, d, e, dtype, seed, marked=None, sharpen=30.0):
    """Random queries, keys and values; with `marked`, the last position's queries point at that key
    (and the key is made long), so that its score stands far out wherever the mask lets it be seen."""
    g = torch.Generator().manual_seed(seed)
    q, k, v = torch.randn(S, H, d, generator=g), torch.randn(S, G, d, generator=g), torch.randn(S, G, e, generator=g)
    if marked is not None:
        k[marked] *= 3.0
        for h in range(H):
            kk = k[marked, h // (H // G)]
            q[S - 1, h] = kk * (sharpen / kk.pow(2).sum()) + 0.05 * q[S - 1, h]
    return q.to(DT[dtype]), k.to(DT[dtype]), v.to(DT[dtype])


KERNELS = [("float32", "float", "all"), ("bfloat16", "float", "all"), ("bfloat16", "matrix cores", "tiles"),
           ("bfloat16", "matrix cores", "singles")]


def _attend(q, kc, vc, bt, positions, how, chunk, scale, H, G, d, e, softcap, sink):
    from sharpinference_amd import ops

    S = int(positions.max()) + 1
    if how == "all":
        return ops.attention_generic(q, kc, vc, bt.to(DEV), torch.zeros(q.shape[0], dtype=torch.int32, device=DEV), positions.to(DEV),
                                     1 if chunk else 0, chunk or 0, scale, H, G, d, e, softcap=softcap, sink=sink)
    assert d == e and ops.decode_attention_ok(q.dtype, d) and ops.prefill_attention_ok(q.dtype, d)
    ctx = _Ctx(positions, tiles=how == "tiles", singles=how == "singles")
    return ops.attention(q, kc, vc, _Group(bt, S), ctx, 1 if chunk else 0, chunk or 0, scale, H, G, d, e, softcap=softcap, sink=sink)


@pytest.mark.parametrize("dtype, kernel, how", KERNELS)
@pytest.mark.parametrize("S, H, G, d, e, chunk, softcap, sink", [
    (70, 4, 2, 64, 64, None, 0.0, True), (200, 8, 2, 96, 96, 64, 50.0, True), (131, 2, 1, 32, 32, 48, 3.0, True),
    (90, 6, 6, 64, 64, 21, 1.5, False), (333, 4, 4, 128, 128, 200, 0.0, False), (50, 4, 2, 12, 20, 16, 6.0, True),
])
def test_attention_with_capped_scores_a_sink_and_chunks(dtype, kernel, how, S, H, G, d, e, chunk, softcap, sink):
    if kernel == "matrix cores" and (d != e or d % 32):
        pytest.skip("the float kernel serves this size")
    q, k, v = _attention_case(S, H, G, d, e, dtype, seed=S)
    scale = 2.5 / math.sqrt(d)                                   # scores large enough that the cap bends them
    kc, vc, bt = _paged(k, v, dtype, seed=S)
    pos = torch.arange(S, dtype=torch.int32)
    out = _attend(q.reshape(S, -1).to(DEV), kc, vc, bt, pos, how, chunk, scale, H, G, d, e, softcap, sink)
    want = P.masked_attention(q.double(), k.double(), v.double(), P.visible(pos.long(), chunk), scale, softcap or None, sink)
    err = _rel_rows(out.reshape(S, -1), want.reshape(S, -1))
    assert float(err.max()) < (2e-6 if dtype == "float32" else 1.5e-2), float(err.max())
    # cap and sink matter at these scores: the plain result without either is far away
    if softcap and softcap < 10:
        other = P.masked_attention(q.double(), k.double(), v.double(), P.visible(pos.long(), chunk), scale, None, sink)
        assert _rel_rms(other.reshape(S, -1), want.reshape(S, -1)) > 0.05
    if sink:
        other = P.masked_attention(q.double(), k.double(), v.double(), P.visible(pos.long(), chunk), scale, softcap or None, False)
        assert _rel_rms(other.reshape(S, -1), want.reshape(S, -1)) > 0.02


@pytest.mark.parametrize("dtype, kernel, how", KERNELS)
@pytest.mark.parametrize("S, chunk, marked, seen", [
    (691, None, 0, True), (691, None, 15, True), (691, None, 16, True), (691, None, 255, True), (691, None, 256, True),
    (691, None, 640, True), (691, None, 689, True),
    (300, 100, 200, True), (300, 100, 199, False), (300, 100, 201, True), (300, 100, 0, False),      # the chunk's first key and the one before it
    (257, 64, 256, True), (257, 64, 255, False), (256, 64, 192, True), (256, 64, 191, False),        # a query that opens a chunk; one that closes it
    (130, 21, 126, True), (130, 21, 125, False), (130, 21, 129, True),                                # chunks that are no multiple of a page
])
def test_one_key_among_hundreds_is_found_or_hidden_as_the_chunk_says(dtype, kernel, how, S, chunk, marked, seen):
    """The last position's queries point at one long key.  Where the mask lets it be seen the result
    is that key's value; where it lies just outside the chunk, the result must not know of it."""
    H, G, d = 4, 2, 64
    q, k, v = _attention_case(S, H, G, d, d, dtype, seed=S + marked, marked=marked)
    kc, vc, bt = _paged(k, v, dtype, seed=marked)
    if how == "tiles":
        rows, pos = q.reshape(S, -1), torch.arange(S, dtype=torch.int32)
    else:
        rows, pos = q[S - 1:].reshape(1, -1), torch.tensor([S - 1], dtype=torch.int32)
    out = _attend(rows.to(DEV), kc, vc, bt, pos, how, chunk, 1.0, H, G, d, d, 40.0, True)[-1:].cpu()
    allpos = torch.arange(S)
    want = P.masked_attention(q.double(), k.double(), v.double(), P.visible(allpos, chunk), 1.0, 40.0, True)[S - 1].reshape(1, -1)
    value = torch.stack([v[marked, h // (H // G)] for h in range(H)]).double().reshape(1, -1)
    if seen:
        assert _rel_rms(want, value) < 0.05                      # the marked key carries the result
    else:
        assert _rel_rms(want, value) > 0.5
    assert _rel_rms(out, want) < (2e-6 if dtype == "float32" else 1.5e-2)


# ---------------------------------------------------------------------------
# the engine
# ---------------------------------------------------------------------------
@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    from sharpinference_amd import load_config
    from sharpinference_amd.weights.loader import write_random_model

    out = {}
    for name in CONFIGS:
        d = str(tmp_path_factory.mktemp("pazatar_" + name))
        write_random_model(load_config(config(name)), d, SEEDS[name], std=0.1, std_by_suffix=STD_BY_SUFFIX)
        out[name] = d
    return out


@functools.lru_cache(maxsize=4)
def _plain_model(d):
    return P.read_config(d), P.load_weights(d, torch.float64)


def _engine(d, dtype, **kw):
    from sharpinference_amd.engine import Engine

    args = dict(dtype=dtype, device=DEV, max_num_seqs=4, kv_tokens=1024, max_model_len=1024)
    args.update(kw)
    return Engine(d, **args)


def _run(eng, reqs, steps, free=True):
    """steps: lists of (request id, number of its next tokens).  Returns per request the logits at
    every position."""
    from sharpinference_amd.engine import StepEntry

    at = {r: 0 for r in reqs}
    logits = {r: [] for r in reqs}
    for step in steps:
        entries = []
        for r, n in step:
            if at[r] == 0:
                eng.add_request(r)
            entries.append(StepEntry(r, reqs[r][at[r]:at[r] + n], list(range(n))))
        out = eng.step(entries).cpu()
        o = 0
        for r, n in step:
            logits[r].append(out[o:o + n])
            o += n
            at[r] += n
            if at[r] == len(reqs[r]) and free:
                eng.free_request(r)
    return {r: torch.cat(v) for r, v in logits.items()}


def _check(d, dtype, reqs, got, what):
    cfg, w = _plain_model(d)
    for r, toks in reqs.items():
        err = _rel_rows(got[r], P.forward(cfg, w, toks))
        if dtype == "float32":
            assert float(err.max()) < 1e-4, f"{what}, request {r}: {float(err.max()):.2e}"
            continue
        tol = _bf16_tol(runs_of(cfg))
        ninth = float(torch.quantile(err, 0.9)) if err.numel() > 1 else float(err.max())
        far = int((err > 2.5 * tol).sum())
        assert ninth < tol and far <= max(1, 0.03 * err.numel()) and float(err.max()) < 0.5, \
            f"{what}, request {r}: ninth decile {ninth:.2e}, {far} rows far out, worst {float(err.max()):.2e} (bound {tol:.2e})"


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


def test_the_files_config_lacks_the_rank_and_the_engine_finds_it(model_dirs):
    d = model_dirs["odd"]
    assert "decay_rank" not in open(os.path.join(d, "config.json")).read()
    eng = _engine(d, "float32")
    assert [l.linear.decay_rank for l in eng.config.layers if l.linear is not None] == [5, 3]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["odd", "even", "wide"])
def test_whole_prompts_portions_and_decoding_agree_with_the_plain_model(model_dirs, name, dtype):
    d = model_dirs[name]
    vocab = CONFIGS[name]["vocab"]
    eng = _engine(d, dtype)
    toks = _tokens(150, vocab, 1)
    ways = {
        "whole": [150],
        "decoded one by one": [1] * 3 + [99] + [1] * 48,          # the first tokens alone, then a long tail through page and chunk borders
        "portions": _cuts(150, [2, 3, 17, 2, 64, 5, 16, 1, 31]),
        "pairs": [2] * 75,
    }
    first = None
    for what, cuts in ways.items():
        got = _run(eng, {what: toks}, [[(what, n)] for n in cuts])
        _check(d, dtype, {what: toks}, got, f"{name} {dtype} {what}")
        if dtype == "float32":
            first = got[what] if first is None else first
            assert _rel_rms(got[what], first) < 1e-5, f"{what}: the cut changes the logits"
    assert eng.runner.graph_replays > 0                           # decode steps ran from graphs, states and all
    eng.cache.check_invariants()
    assert not eng.cache.requests


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["odd", "wide"])
def test_a_long_prompt_is_walked_in_segments_and_agrees_with_its_portions(model_dirs, name, dtype, monkeypatch):
    """700 tokens in one step: the linear-attention layers walk them in segments of 128 side by side;
    the same tokens in portions of 100 are walked whole, portion by portion."""
    from sharpinference_amd import ops

    calls = {"segments": 0, "whole": 0}
    walk = ops.gla_walk

    def counted(*a, segments=None, **kw):
        calls["segments" if segments is not None else "whole"] += 1
        return walk(*a, segments=segments, **kw)

    monkeypatch.setattr(ops, "gla_walk", counted)
    d = model_dirs[name]
    toks = _tokens(700, CONFIGS[name]["vocab"], 8)
    eng = _engine(d, dtype, kv_tokens=2048)
    whole = _run(eng, {"w": toks}, [[("w", 700)]])
    assert calls["segments"] > 0 and calls["whole"] == 0
    _check(d, dtype, {"w": toks}, whole, f"{name} {dtype} 700 tokens at once")
    calls["segments"] = 0
    parts = _run(eng, {"p": toks}, [[("p", 100)] for _ in range(7)])
    assert calls["segments"] == 0 and calls["whole"] > 0
    _check(d, dtype, {"p": toks}, parts, f"{name} {dtype} 700 tokens in portions")
    if dtype == "float32":
        assert _rel_rms(whole["w"], parts["p"]) < 1e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_first_tokens_and_a_long_decoded_tail(model_dirs, dtype):
    """Every token from the first decoded alone: 260 steps, through every chunk edge of every layer
    (chunks of 24 and 21 keys; the convolution's tail starts from zeros), replayed from graphs."""
    d = model_dirs["odd"]
    toks = _tokens(260, CONFIGS["odd"]["vocab"], 7)
    eng = _engine(d, dtype)
    got = _run(eng, {"x": toks}, [[("x", 1)] for _ in toks])
    _check(d, dtype, {"x": toks}, got, f"decoded from the first token, {dtype}")
    assert eng.runner.graph_replays >= 250
    # pages behind the chunks went back to their pools on the way
    assert all(g.pool.num_free == g.pool.num_pages for g in eng.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["odd", "even"])
def test_unequal_requests_in_one_batch_give_what_each_gives_alone(model_dirs, name, dtype):
    d = model_dirs[name]
    vocab = CONFIGS[name]["vocab"]
    reqs = {"a": _tokens(90, vocab, 2), "b": _tokens(37, vocab, 3), "c": _tokens(130, vocab, 4), "d": _tokens(5, vocab, 5)}
    steps = [[("a", 29), ("b", 2)], [("a", 1), ("b", 33), ("c", 64)], [("c", 2), ("a", 1), ("d", 5), ("b", 1)],
             [("a", 59), ("c", 1), ("b", 1)], [("c", 63)]]
    eng = _engine(d, dtype)
    got = _run(eng, reqs, steps)
    _check(d, dtype, reqs, got, f"mixed {dtype}")
    if dtype == "float32":
        for r, toks in reqs.items():
            alone = _run(eng, {r: toks}, [[(r, len(toks))]])
            assert _rel_rms(got[r], alone[r]) < 1e-5, f"{r}: the batch changes the logits"
    eng.cache.check_invariants()


def test_pages_and_slots_are_given_back_and_used_again(model_dirs):
    """Two state slots and a pool of a dozen pages serve ten requests in turn: a state or a tail
    that a request before left in its slot, or a key in a page used again, would show."""
    d = model_dirs["even"]
    vocab = CONFIGS["even"]["vocab"]
    eng = _engine(d, "float32", max_num_seqs=2, kv_tokens=192, max_model_len=160, max_tokens_per_step=64)
    slots = set()
    allocs = 0
    for i in range(5):
        a, b = f"a{i}", f"b{i}"
        reqs = {a: _tokens(100 + i, vocab, 10 + i), b: _tokens(60 - i, vocab, 20 + i)}
        steps = [[(a, 40), (b, 3)], [(a, 60 + i), (b, 57 - i - 1)], [(b, 1)]]
        eng.add_request(a), eng.add_request(b)
        slots |= {eng.cache.requests[a].state_slot, eng.cache.requests[b].state_slot}
        eng.free_request(a), eng.free_request(b)
        got = _run(eng, reqs, steps)
        _check(d, "float32", reqs, got, f"round {i}")
        eng.cache.check_invariants()
    for g in eng.cache.groups:
        assert g.pool.total_allocs > 2 * g.pool.num_pages and g.pool.num_free == g.pool.num_pages
    assert len(slots) == 2


def test_what_the_design_adds_would_show_if_left_out(model_dirs):
    """The weights of these tests make each mechanism matter: the plain model without it is far
    from the engine, the plain model with it is not."""
    d = model_dirs["odd"]
    cfg, w = _plain_model(d)
    toks = _tokens(80, CONFIGS["odd"]["vocab"], 6)
    eng = _engine(d, "float32")
    got = _run(eng, {"x": toks}, [[("x", 50)], [("x", 30)]])["x"]
    assert _rel_rms(got, P.forward(cfg, w, toks)) < 1e-4

    def changed(**kw):
        c = json.loads(json.dumps(cfg))
        ww = dict(w)
        if kw.get("no_loop_vectors"):
            ww["loop.step"] = torch.zeros_like(w["loop.step"])
        if kw.get("one_pass"):
            c["loop"]["times"] = 1
        if kw.get("no_cap"):
            c["layers"][1]["mixer"]["left"].pop("softcap")
        if kw.get("no_chunks"):
            for l in c["layers"]:
                (l["mixer"].get("left") or l["mixer"]).pop("mask", None)
        if kw.get("no_scaling"):
            for l in c["layers"]:
                m = l["mixer"].get("left") or l["mixer"]
                if m.get("rot"):
                    m["rot"].pop("scaling", None)
        if kw.get("identity_conv"):
            for k in w:
                if k.endswith(".conv"):
                    ww[k] = torch.zeros_like(w[k])
                    ww[k][:, -1] = 1.0
        if kw.get("no_decay"):
            for k in w:
                if k.endswith(".a2.b"):
                    ww[k] = torch.full_like(w[k], 40.0)
                if k.endswith(".a2"):
                    ww[k] = torch.zeros_like(w[k])
        return float(_rel_rows(got, P.forward(c, ww, toks)).max())

    for what in ("no_loop_vectors", "one_pass", "no_cap", "no_chunks", "no_scaling", "identity_conv", "no_decay"):
        assert changed(**{what: True}) > 5e-3, what


@pytest.mark.parametrize("name", ["odd", "even", "wide"])
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
