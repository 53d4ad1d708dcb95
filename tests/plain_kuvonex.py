"""A plain, slow Kuvonex decoder: whole sequences, no cache, one function a mechanism.

The yardstick of the Kuvonex tests.  It shares no code with the package: it takes ``config.json``
as a raw dict and weights as a ``{name: tensor}`` dict and computes with dense tensor arithmetic
on the CPU, keys and values expanded per head from the latent (the engine never forms them).

Notation: T tokens, W the model width, H heads, dn / dr the unrotated / rotated width of a
query or key head, dv the width of a value head, R the latent's width, E experts.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence, Tuple

import torch

GROUP_TOP = 2      # a group of experts is ranked by the sum of this many of its best choice scores


def read_config(model_dir: str) -> dict:
    with open(os.path.join(model_dir, "config.json")) as f:
        return json.load(f)


def load_weights(model_dir: str, dtype=torch.float32) -> Dict[str, torch.Tensor]:
    """Every tensor of model.safetensors, floats widened to `dtype` (own reader: 8 bytes of
    length, a JSON header, raw data)."""
    path = os.path.join(model_dir, "model.safetensors")
    with open(path, "rb") as f:
        n = int.from_bytes(f.read(8), "little")
        header = json.loads(f.read(n))
        base = 8 + n
        out = {}
        kinds = {"BF16": torch.bfloat16, "F32": torch.float32, "F16": torch.float16, "I32": torch.int32, "I64": torch.int64}
        for name, e in header.items():
            if name == "__metadata__":
                continue
            a, b = e["data_offsets"]
            f.seek(base + a)
            t = torch.frombuffer(bytearray(f.read(b - a)), dtype=kinds[e["dtype"]]).reshape(e["shape"])
            out[name] = t.to(dtype) if t.dtype.is_floating_point else t.to(torch.int64)
    return out


# ----------------------------------------------------------------------------
# the small pieces
# ----------------------------------------------------------------------------
def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) along the last axis."""
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * w


def embed(tokens: Sequence[int], table: torch.Tensor, scale: float) -> torch.Tensor:
    return table[torch.as_tensor(list(tokens), dtype=torch.long)] * scale


def rotate(v: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """Rotary positions on the first `dims` elements of the last axis, element 2i paired with
    2i + 1: (a, b) -> (a cos t - b sin t, b cos t + a sin t), t = p * base^(-2i / dims).
    v [T, ..., n], positions [T]."""
    out = v.clone()
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    ang = positions.to(torch.float64)[:, None] * freq[None, :]                      # [T, half]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [half]
    cos, sin = ang.cos().to(v.dtype).reshape(shape), ang.sin().to(v.dtype).reshape(shape)
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    out[..., 0:dims:2] = a * cos - b * sin
    out[..., 1:dims:2] = b * cos + a * sin
    return out


def latent_of(h: torch.Tensor, w_dkv: torch.Tensor, norm_w: torch.Tensor, eps: float, rank: int,
              positions: torch.Tensor, base: float, dims: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """What a latent layer keeps of a token: c [T, R] = rms_norm(first R rows of W_dkv h) and the
    one rotated key part [T, dr] all heads share (the remaining rows, rotated, not normed)."""
    d = h @ w_dkv.T
    return rms_norm(d[:, :rank], norm_w, eps), rotate(d[:, rank:], positions, base, dims)


def sink_attention(qn: torch.Tensor, qr: torch.Tensor, kn: torch.Tensor, kr: torch.Tensor, v: torch.Tensor,
                   sink: torch.Tensor, scale: float, q_pos: torch.Tensor, k_pos: torch.Tensor) -> torch.Tensor:
    """Causal attention whose softmax has one more term in the denominator, exp(sink_h), with
    no key and no value.  qn [T, H, dn], qr [T, H, dr], kn [S, H, dn], kr [S, dr] (shared by the
    heads), v [S, H, dv] -> [T, H, dv]."""
    s = (torch.einsum("thd,shd->hts", qn, kn) + torch.einsum("thd,sd->hts", qr, kr)) * scale
    s = s.masked_fill(k_pos[None, None, :] > q_pos[None, :, None], float("-inf"))
    m = torch.maximum(s.max(dim=-1).values, sink[:, None])                           # [H, T]
    e = torch.exp(s - m[..., None])
    den = e.sum(dim=-1) + torch.exp(sink[:, None] - m)
    return torch.einsum("hts,shd->thd", e / den[..., None], v)


def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mx: dict, eps: float,
                     positions: torch.Tensor, kept: Optional[Tuple[torch.Tensor, torch.Tensor]] = None):
    """The mixer.  `kept` = (c, rotated key part) of the layer named by kv_from, else they are made
    here.  Returns (output [T, W], (c, rotated key part))."""
    T = h.shape[0]
    H, dn, dr, dv, R = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
    base, dims = float(mx["rot"]["base"]), int(mx["rot"]["dims"])
    q = (h @ w[p + "q"].T).reshape(T, H, dn + dr)
    qn, qr = q[..., :dn], rotate(q[..., dn:], positions, base, dims)
    if kept is None:
        kept = latent_of(h, w[p + "dkv"], w[p + "dkv.norm"], eps, R, positions, base, dims)
    c, kr = kept
    kn = (c @ w[p + "uk"].T).reshape(-1, H, dn)
    v = (c @ w[p + "uv"].T).reshape(-1, H, dv)
    o = sink_attention(qn, qr, kn, kr, v, w[p + "sink"], float(mx["scale"]), positions, positions)
    o = o.reshape(T, H * dv) * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T, kept


def route(h: torch.Tensor, w_router: torch.Tensor, correction: torch.Tensor, router: dict, ids=None):
    """Picks and weights.  s = sigmoid(W_router h); experts are chosen by s + correction, among the
    experts of the `keep` best groups only (a group's rank: the sum of its GROUP_TOP largest
    choice scores); the weights are s of the chosen, as they are.  Returns ids [T, top] (best
    first), weights [T, top].  With `ids` given, only the weights of those picks are made."""
    E, top = int(router["experts"]), int(router["top"])
    s = torch.sigmoid(h @ w_router.T)
    if ids is not None:
        return ids, s.gather(1, ids)
    choice = s + correction
    groups = router.get("groups")
    if groups:
        n, keep = int(groups["count"]), int(groups["keep"])
        per = E // n
        g = choice.reshape(-1, n, per)
        rank = g.topk(min(GROUP_TOP, per), dim=-1).values.sum(dim=-1)                # [T, n]
        best = rank.topk(keep, dim=-1).indices
        allowed = torch.zeros_like(rank, dtype=torch.bool).scatter_(1, best, True)
        choice = choice.masked_fill(~allowed.repeat_interleave(per, dim=1), float("-inf"))
    ids = choice.topk(top, dim=-1).indices
    return ids, s.gather(1, ids)


def expert(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    g = h @ w[p + "gate"].T
    return ((g * torch.sigmoid(g)) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def moe(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mlp: dict, picks=None) -> torch.Tensor:
    """The weighted sum of the chosen experts' outputs (`picks`: expert ids [T, top] that replace the
    router's choice; their weights are still the router's scores)."""
    ids, wts = route(h, w[p + "router"], w[p + "correction"], mlp["router"], picks)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, s in zip(ids[t].tolist(), wts[t]):
            out[t] += s * expert(h[t:t + 1], w, f"{p}e{e}.")[0]
    return out


# ----------------------------------------------------------------------------
# the whole model
# ----------------------------------------------------------------------------
def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: Sequence[int], picks: Optional[dict] = None,
            want_layers: bool = False):
    """Logits [T, vocab] of a whole sequence (and the residual stream after every layer, if asked).
    A layer is x += norm1(mixer(x)); x += norm2(ff(x)): the branches read x itself, the norms sit
    on their outputs.  `picks` {layer: ids [T, top]} replaces the routers' choices."""
    eps = float(cfg["norm"]["eps"])
    x = embed(tokens, w["embed"], float(cfg["embedding"]["scale"]))
    pos = torch.arange(len(tokens))
    kept: Dict[int, tuple] = {}
    after: List[torch.Tensor] = []
    for i, layer in enumerate(cfg["layers"]):
        if layer["type"] != "latent_attention":
            raise ValueError(f"layer type {layer['type']!r}")
        p = f"l{i}."
        src = layer["mixer"].get("kv_from")
        y, kept[i] = latent_attention(x, w, p + "mix.", layer["mixer"], eps, pos, None if src is None else kept[src])
        x = x + rms_norm(y, w[p + "norm1"], eps)
        if layer.get("mlp") is not None:
            y = moe(x, w, p + "mlp.", layer["mlp"], None if picks is None else picks.get(i))
            x = x + rms_norm(y, w[p + "norm2"], eps)
        after.append(x)
    logits = rms_norm(x, w["final.norm"], eps) @ w["head"].T
    return (logits, torch.stack(after)) if want_layers else logits


def generate(cfg: dict, w: Dict[str, torch.Tensor], prompt: Sequence[int], n: int) -> List[int]:
    """Greedy continuation by whole-sequence recomputation (the lowest index wins a tie)."""
    toks, out = list(prompt), []
    for _ in range(n):
        nxt = int(torch.argmax(forward(cfg, w, toks)[-1]))
        out.append(nxt)
        toks.append(nxt)
    return out
