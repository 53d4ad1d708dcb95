"""The latent attention mixer: keys and values of all heads kept as one low-rank row per token."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..cache.spec import KVSpec, WINDOW_NONE
from ..ops.profile import section
from .attention import _WORK_LISTS
from .base import LayerCache, ParamSpec, Part, StepContext, TensorSource


class LatentAttention(Part):
    """Attention whose cache holds, per token, a latent c [rank] and one rotated key part [dr]
    shared by all heads, instead of per-head keys and values.

    With h the input: q = W_q h, per head [dn unrotated | dr rotated]; W_dkv h gives rank + dr
    elements, the first rank RMS-normed (weight ``dkv.norm``) into c, the last dr rotated into the
    shared key part.  A head's unrotated key is W_uk c and its value W_uv c; its score against a
    key is (q_n . W_uk c + q_r . k_r) * scale.  Neither keys nor values are ever formed: the
    unrotated query is taken through W_uk first (q_n^T W_uk) c, so that all heads attend over the
    cached rows [c | k_r] themselves (the score is one dot product over rank + dr elements, the
    weighted sum of the rows' first rank elements is taken through W_uv afterwards).  Softmax in
    float, with ``sink``: one learned term exp(sink_h) more in the denominator, without key or
    value.  With ``gate`` the heads' outputs are multiplied by sigmoid(W_g h) before W_o.

    ``own_latent=False``: the layer has no W_dkv and attends over the rows another layer stored
    (the schedule hands it that layer's cache with ``write=False``).  ``rotary``: any object with
    ``table(device)`` (float32 frequencies of the rotated pairs (2i, 2i + 1), at most dr / 2).
    """

    NAMES = {"q": "q", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "sink": "sink", "g": "g", "o": "o"}

    def __init__(self, hidden: int, num_heads: int, nope_dim: int, rope_dim: int, v_dim: int, rank: int, rotary,
                 norm_eps: float, scale: float, sink: bool = True, gate: bool = True, own_latent: bool = True,
                 window_kind: int = WINDOW_NONE, window: int = 0, names: Optional[Dict[str, str]] = None):
        if rank < 1 or rank > ops.LATENT_MAX_RANK:
            raise ValueError(f"a latent of {rank} elements is not taken: 1 to {ops.LATENT_MAX_RANK}")
        if min(num_heads, nope_dim, rope_dim, v_dim) < 1:
            raise ValueError("heads and head sizes must be positive")
        if rotary is not None and (rotary.pair_layout != "interleaved" or rotary.rotary_dim > rope_dim):
            raise ValueError("the rotated part takes interleaved pairs, at most as many as it is wide")
        self.hidden, self.nh, self.dn, self.dr, self.dv, self.rank = (int(hidden), int(num_heads), int(nope_dim),
                                                                     int(rope_dim), int(v_dim), int(rank))
        self.rotary, self.eps, self.scale = rotary, float(norm_eps), float(scale)
        self.has_sink, self.has_gate, self.own_latent = bool(sink), bool(gate), bool(own_latent)
        self.window_kind, self.window = int(window_kind), int(window)
        self.names = {**self.NAMES, **(names or {})}
        self.w_in = None                                   # [q | g | dkv] rows: one product of the input
        self.w_uk_t: Optional[torch.Tensor] = None         # [heads, rank, dn]: W_uk per head, transposed
        self.w_uv: Optional[torch.Tensor] = None           # [heads, dv, rank]
        self.w_o = None
        self.w_norm: Optional[torch.Tensor] = None         # float32 [rank]
        self.w_sink: Optional[torch.Tensor] = None         # float32 [heads]

    # -- what it needs --------------------------------------------------------
    def step_planners(self):
        return (_WORK_LISTS,)

    def cache_spec(self) -> KVSpec:
        return KVSpec(1, self.rank + self.dr, self.window_kind, self.window, self.rank, values_in_keys=True)

    @property
    def q_dim(self) -> int:
        return self.nh * (self.dn + self.dr)

    @property
    def o_dim(self) -> int:
        return self.nh * self.dv

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        n = self.names
        specs = {
            prefix + n["q"]: ParamSpec((self.q_dim, self.hidden)),
            prefix + n["uk"]: ParamSpec((self.nh * self.dn, self.rank)),
            prefix + n["uv"]: ParamSpec((self.o_dim, self.rank)),
            prefix + n["o"]: ParamSpec((self.hidden, self.o_dim)),
        }
        if self.own_latent:
            specs[prefix + n["dkv"]] = ParamSpec((self.rank + self.dr, self.hidden))
            specs[prefix + n["dkv_norm"]] = ParamSpec((self.rank,), "norm_weight")
        if self.has_sink:
            specs[prefix + n["sink"]] = ParamSpec((self.nh,))
        if self.has_gate:
            specs[prefix + n["g"]] = ParamSpec((self.o_dim, self.hidden))
        return specs

    def load(self, prefix: str, source: TensorSource) -> None:
        n = self.names
        parts = [source.get(prefix + n["q"])]
        if self.has_gate:
            parts.append(source.get(prefix + n["g"]))
        if self.own_latent:
            parts.append(source.get(prefix + n["dkv"]))
            self.w_norm = source.get(prefix + n["dkv_norm"]).float().contiguous()
        dt = torch.float32 if any(p.dtype == torch.float32 for p in parts) else parts[0].dtype
        fused = torch.empty(sum(p.shape[0] for p in parts), self.hidden, dtype=dt, device=parts[0].device)
        o = 0
        for p in parts:
            fused[o:o + p.shape[0]].copy_(p)
            o += p.shape[0]
        self.w_in = ops.pack_weight(fused)
        uk = source.get(prefix + n["uk"]).to(dt)
        self.w_uk_t = uk.view(self.nh, self.dn, self.rank).transpose(1, 2).contiguous()
        self.w_uv = source.get(prefix + n["uv"]).to(dt).view(self.nh, self.dv, self.rank).contiguous()
        self.w_o = ops.pack_weight(source.get(prefix + n["o"]))
        if self.has_sink:
            self.w_sink = source.get(prefix + n["sink"]).float().contiguous()

    # -- compute --------------------------------------------------------------
    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        g = cache.group
        T = x.shape[0]
        D = self.rank + self.dr
        width = 2 if ctx.act_dtype == torch.bfloat16 else 4
        n_in = self.w_in.shape[0]
        g_off = self.q_dim
        kv_off = self.q_dim + (self.o_dim if self.has_gate else 0)
        with section("q|g|dkv", nbytes=width * n_in * (self.hidden + T) + width * T * self.hidden, flops=2.0 * T * self.hidden * n_in):
            proj = ops.linear(x, self.w_in, ctx.act_dtype)
        store = self.own_latent and cache.write
        if self.own_latent and not cache.write:
            raise ValueError("a latent layer with a down projection of its own must own its cache")
        q_full = torch.empty(T, self.nh * D, dtype=ctx.act_dtype, device=x.device)
        inv_freq = self.rotary.table(x.device) if self.rotary is not None else None
        with section("latent + rotary + cache write", nbytes=width * T * (2 * self.nh * self.dr + 2 * D)):
            ops.latent_prep(proj, 0, kv_off if store else None, q_full, cache.k, g.slot_mapping if store else None,
                            ctx.positions, inv_freq, self.w_norm, self.eps, self.nh, self.dn, self.dr, self.rank)
        with section("q through uk", nbytes=width * (self.nh * self.dn * self.rank + T * self.nh * (self.dn + self.rank)),
                     flops=2.0 * T * self.nh * self.dn * self.rank):
            ops.head_gemm(proj, 0, self.dn + self.dr, self.w_uk_t, q_full, 0, D)
        with section("attention", nbytes=lambda: self._keys_held(ctx) * D * width + T * self.nh * (D + self.rank) * width,
                     flops=lambda: 2.0 * self._keys_read(ctx) * self.nh * (D + self.rank)):
            o_lat = ops.attention_latent(q_full, cache.k, g, ctx, self.scale, self.nh, self.rank, self.dr, sink=self.w_sink,
                                         window_kind=self.window_kind, window=self.window)
        o = torch.empty(T, self.o_dim, dtype=ctx.act_dtype, device=x.device)
        with section("uv + gate", nbytes=width * (self.o_dim * self.rank + T * (self.nh * self.rank + 2 * self.o_dim)),
                     flops=2.0 * T * self.o_dim * self.rank):
            ops.head_gemm(o_lat, 0, self.rank, self.w_uv, o, 0, self.dv, gate=proj if self.has_gate else None, gate_off=g_off)
        with section("o", nbytes=width * self.hidden * (self.o_dim + T) + width * T * self.o_dim, flops=2.0 * T * self.hidden * self.o_dim):
            return ops.linear(o, self.w_o, ctx.act_dtype)

    def _keys_read(self, ctx: StepContext) -> int:
        spec = self.cache_spec()
        return sum(p - spec.first_visible(p) + 1 for s, n in zip(ctx.entry_starts, ctx.entry_lens) for p in range(s, s + n))

    def _keys_held(self, ctx: StepContext) -> int:
        spec = self.cache_spec()
        return sum(s + n - spec.first_visible(s) for s, n in zip(ctx.entry_starts, ctx.entry_lens))
