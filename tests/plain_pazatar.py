"""A plain, slow Pazatar decoder: whole sequences, no cache, one function a mechanism.

The yardstick of the Pazatar tests.  It shares no code with the package: ``config.json`` as a raw
dict, weights as a ``{name: tensor}`` dict, dense tensor arithmetic on the CPU (float64 unless
told otherwise), every key and every state of a sequence recomputed from its first token.

Notation: T tokens, W the model width, H query heads, G key/value heads, d the width of a query
or key head, e the width of a value head, n the taps of a short convolution.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch

YARN_MAGNITUDE_SLOPE = 0.1     # cos and sin of a YaRN-scaled rotation are multiplied by 0.1 ln(factor) + 1


def read_config(model_dir: str) -> dict:
    with open(os.path.join(model_dir, "config.json")) as f:
        return json.load(f)


def load_weights(model_dir: str, dtype=torch.float64) -> Dict[str, torch.Tensor]:
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


def relu_squared(z: torch.Tensor) -> torch.Tensor:
    return torch.relu(z).pow(2)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def short_convolution(u: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """y_t = sum_j w[:, j] * u_(t - n + 1 + j), zeros before the first token.  u [T, C], w [C, n]."""
    T, C = u.shape
    n = w.shape[1]
    padded = torch.cat([u.new_zeros(n - 1, C), u], dim=0)
    y = u.new_zeros(T, C)
    for j in range(n):
        y = y + padded[j:j + T] * w[:, j]
    return y


# ----------------------------------------------------------------------------
# rotary positions
# ----------------------------------------------------------------------------
def plain_frequencies(base: float, dims: int) -> List[float]:
    return [base ** (-2.0 * i / dims) for i in range(dims // 2)]


def stretched_frequencies(base: float, dims: int, s: dict) -> List[float]:
    """The Llama 3.1 rule: short wavelengths stay, long ones are divided by the factor, those
    between are blended.  s: factor, low, high, original."""
    out = []
    for f in plain_frequencies(base, dims):
        wavelength = 2.0 * math.pi / f
        if wavelength < s["original"] / s["high"]:
            out.append(f)
        elif wavelength > s["original"] / s["low"]:
            out.append(f / s["factor"])
        else:
            t = (s["original"] / wavelength - s["low"]) / (s["high"] - s["low"])
            out.append((1.0 - t) * f / s["factor"] + t * f)
    return out


def yarn_frequencies(base: float, dims: int, s: dict) -> List[float]:
    """YaRN: pair i is interpolated by ramp_i, which rises from 0 at the pair that turns `fast`
    times within the original context to 1 at the pair that turns `slow` times."""
    def pair_of(turns: float) -> float:
        return dims * math.log(s["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_of(s["fast"])), 0)
    hi = min(math.ceil(pair_of(s["slow"])), dims - 1)
    out = []
    for i, f in enumerate(plain_frequencies(base, dims)):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / s["factor"] * ramp + f * (1.0 - ramp))
    return out


def yarn_magnitude(s: dict) -> float:
    return YARN_MAGNITUDE_SLOPE * math.log(s["factor"]) + 1.0


def rotate(x: torch.Tensor, positions: torch.Tensor, freqs: Sequence[float], layout: str, magnitude: float = 1.0) -> torch.Tensor:
    """Rotary positions on the first 2 * len(freqs) elements of the last axis of x [T, heads, d]:
    the pair (a, b) -> (a cos t - b sin t, b cos t + a sin t) * magnitude, t = p * f_i.  layout
    "interleaved": a, b = elements 2i, 2i + 1; "half": elements i, i + dims / 2."""
    half = len(freqs)
    dims = 2 * half
    ang = positions.to(torch.float64)[:, None] * torch.tensor(list(freqs), dtype=torch.float64)[None, :]
    cos = (ang.cos() * magnitude).to(x.dtype)[:, None, :]
    sin = (ang.sin() * magnitude).to(x.dtype)[:, None, :]
    out = x.clone()
    if layout == "interleaved":
        a, b = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = a * cos - b * sin
        out[..., 1:dims:2] = b * cos + a * sin
    elif layout == "half":
        a, b = x[..., :half], x[..., half:dims]
        out[..., :half] = a * cos - b * sin
        out[..., half:dims] = b * cos + a * sin
    else:
        raise ValueError(layout)
    return out


# ----------------------------------------------------------------------------
# attention over the keys a mask admits
# ----------------------------------------------------------------------------
def visible(positions: torch.Tensor, chunk: Optional[int]) -> torch.Tensor:
    """[T, T] bool: query i sees key j <= i, and with a chunk size only inside its own chunk
    (chunks counted from position 0)."""
    i, j = positions[:, None], positions[None, :]
    ok = j <= i
    if chunk:
        ok = ok & (torch.div(i, chunk, rounding_mode="floor") == torch.div(j, chunk, rounding_mode="floor"))
    return ok


def masked_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: torch.Tensor, scale: float,
                     softcap: Optional[float] = None, sink: bool = False) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, e] -> [T, H, e].  Query head h reads key/value head
    h // (H / G).  softcap: s <- cap tanh(s / cap).  sink: one more term exp(0) in the softmax's
    denominator, with no value."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = q.new_zeros(T, H, v.shape[2])
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        s = s.masked_fill(~mask, float("-inf"))
        m = s.max(dim=-1, keepdim=True).values
        if sink:
            m = torch.clamp(m, min=0.0)
        e = torch.exp(s - m)
        den = e.sum(dim=-1, keepdim=True)
        if sink:
            den = den + torch.exp(-m)
        out[:, h] = (e / den) @ v[:, g]
    return out


def attention_mixer(h: torch.Tensor, positions: torch.Tensor, p: Dict[str, torch.Tensor], pre: str, m: dict, eps: float) -> torch.Tensor:
    """The mixer 'attention': the values are the keys as projected; query and key are normed over
    their whole projections, rotated on interleaved pairs with YaRN frequencies."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = h @ p[pre + "q"].T
    k = h @ p[pre + "k"].T
    v = k.reshape(T, G, d)
    q = rms_norm(q, p[pre + "q.norm"], eps).reshape(T, H, d)
    k = rms_norm(k, p[pre + "k.norm"], eps).reshape(T, G, d)
    rot = m.get("rot")
    if rot:
        s = rot.get("scaling")
        freqs = yarn_frequencies(rot["base"], rot["dims"], s) if s else plain_frequencies(rot["base"], rot["dims"])
        mag = yarn_magnitude(s) if s else 1.0
        q, k = rotate(q, positions, freqs, "interleaved", mag), rotate(k, positions, freqs, "interleaved", mag)
    mask = visible(positions, (m.get("mask") or {}).get("size"))
    o = masked_attention(q, k, v, mask, m["scale"])
    return o.reshape(T, H * v.shape[2]) @ p[pre + "o"].T


def left_mixer(h: torch.Tensor, positions: torch.Tensor, p: Dict[str, torch.Tensor], pre: str, m: dict, eps: float) -> torch.Tensor:
    """Softmax attention with short convolutions behind the projections, a per-head norm, rotation
    on split halves with stretched frequencies, capped scores and a sink."""
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = h @ p[pre + "q"].T, h @ p[pre + "k"].T, h @ p[pre + "v"].T
    if m.get("conv"):
        q, k, v = (short_convolution(u, p[pre + n + ".conv"]) for u, n in ((q, "q"), (k, "k"), (v, "v")))
    q = rms_norm(q.reshape(T, H, d), p[pre + "q.norm"], eps)
    k = rms_norm(k.reshape(T, G, d), p[pre + "k.norm"], eps)
    v = v.reshape(T, G, e)
    rot = m.get("rot")
    if rot:
        s = rot.get("scaling")
        freqs = stretched_frequencies(rot["base"], rot["dims"], s) if s else plain_frequencies(rot["base"], rot["dims"])
        q, k = rotate(q, positions, freqs, "half"), rotate(k, positions, freqs, "half")
    mask = visible(positions, (m.get("mask") or {}).get("size"))
    o = masked_attention(q, k, v, mask, m["scale"], softcap=m.get("softcap"), sink=True)
    return o.reshape(T, H * e) @ p[pre + "o"].T


def decays(h: torch.Tensor, p: Dict[str, torch.Tensor], pre: str, tau: float) -> torch.Tensor:
    """alpha = sigmoid(z)^(1 / tau), z = W_a2 (W_a1 h) + b: one decay per key channel, in (0, 1)."""
    z = (h @ p[pre + "a1"].T) @ p[pre + "a2"].T + p[pre + "a2.b"]
    return torch.exp(torch.nn.functional.logsigmoid(z) / tau)


def gated_recurrence(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, alpha: torch.Tensor,
                     state: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Per head S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, token by token.
    q, k, alpha [T, H, d]; v [T, H, e]; state [H, d, e] (zeros unless given) -> o [T, H, e]."""
    T, H, d = q.shape
    S = q.new_zeros(H, d, v.shape[2]) if state is None else state.clone()
    out = q.new_zeros(T, H, v.shape[2])
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hde,hd->he", S, q[t])
    return out


def right_mixer(h: torch.Tensor, p: Dict[str, torch.Tensor], pre: str, m: dict, eps: float) -> torch.Tensor:
    """Gated linear attention: the recurrence above, a per-head norm on its outputs, a SiLU gate."""
    T = h.shape[0]
    H, d, e = m["heads"], m["dim"], m["vdim"]
    q = (h @ p[pre + "q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ p[pre + "k"].T).reshape(T, H, d)
    v = (h @ p[pre + "v"].T).reshape(T, H, e)
    alpha = decays(h, p, pre, m["tau"]).reshape(T, H, d)
    o = gated_recurrence(q, k, v, alpha)
    o = rms_norm(o, p[pre + "norm"], eps).reshape(T, H * e)
    return (o * silu(h @ p[pre + "g"].T)) @ p[pre + "o"].T


def parallel_mixer(h: torch.Tensor, positions: torch.Tensor, p: Dict[str, torch.Tensor], pre: str, m: dict, eps: float) -> torch.Tensor:
    """Two mixers on the same input; half the sum of their outputs, each normed over the width."""
    left = left_mixer(h, positions, p, pre + "left.", m["left"], eps)
    right = right_mixer(h, p, pre + "right.", m["right"], eps)
    return 0.5 * (rms_norm(left, p[pre + "left.out"], eps) + rms_norm(right, p[pre + "right.out"], eps))


def dense_feed_forward(h: torch.Tensor, p: Dict[str, torch.Tensor], pre: str) -> torch.Tensor:
    return relu_squared(h @ p[pre + "up"].T) @ p[pre + "down"].T


# ----------------------------------------------------------------------------
# the whole model
# ----------------------------------------------------------------------------
def layer_order(cfg: dict) -> List[tuple]:
    """(layer, pass or None) in the order the layers run: layers start .. stop - 1 `times` times in
    a row, the others once."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    order = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        order += [(i, t) for i in range(loop["start"], loop["stop"])]
    return order + [(i, None) for i in range(loop["stop"], n)]


def run_layer(x: torch.Tensor, positions: torch.Tensor, p: Dict[str, torch.Tensor], i: int, layer: dict, eps: float) -> torch.Tensor:
    pre = f"l{i}."
    h = rms_norm(x, p[pre + "norm1"], eps)
    if layer["type"] == "attention":
        y = attention_mixer(h, positions, p, pre + "mix.", layer["mixer"], eps)
    elif layer["type"] == "parallel":
        y = parallel_mixer(h, positions, p, pre + "mix.", layer["mixer"], eps)
    else:
        raise ValueError(layer["type"])
    x = x + rms_norm(y, p[pre + "norm1b"], eps)
    if layer.get("mlp"):
        y = dense_feed_forward(rms_norm(x, p[pre + "norm2"], eps), p, pre + "mlp.")
        x = x + rms_norm(y, p[pre + "norm2b"], eps)
    return x


def forward(cfg: dict, p: Dict[str, torch.Tensor], tokens: Sequence[int], layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of a whole sequence.  layers_out (a list) receives the residual sum after
    every layer run."""
    eps = cfg["norm"]["eps"]
    x = p["embed"][torch.as_tensor(list(tokens), dtype=torch.long)]
    positions = torch.arange(len(tokens))
    loop = cfg.get("loop")
    for i, t in layer_order(cfg):
        if t is not None and i == loop["start"]:
            x = x + p["loop.step"][t]
        x = run_layer(x, positions, p, i, cfg["layers"][i], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, p["final.norm"], eps) @ p["embed"].T


def generate(cfg: dict, p: Dict[str, torch.Tensor], prompt: Sequence[int], n_new: int) -> List[int]:
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(forward(cfg, p, toks)[-1].argmax()))
    return toks[len(prompt):]
