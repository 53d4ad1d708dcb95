"""Pazatar: a decoder whose layers hold either softmax attention or softmax attention beside gated
linear attention, each branch between a norm before and a norm after it, a stretch of the layers
run several times, assembled from config.json layer by layer.

* embedding rows; the head is the embedding table;
* every layer x += norm1b(mixer(norm1(x))), then x += norm2b(ff(norm2(x))) where it has a
  feed-forward (down(relu(up h)^2));
* 'attention' layers: grouped-query attention whose values are the keys as projected; query and
  key each RMS-normed over their whole projection with learned weights, then rotated on
  interleaved pairs with YaRN frequencies; chunked mask;
* 'parallel' layers: two mixers on the same input, their outputs each normed over the width and
  averaged.  Left: attention with short causal convolutions behind q, k and v, a per-head norm with
  shared weights, rotation on split halves of the leading elements with stretched wavelengths,
  capped scores, a chunked mask and a sink of score 0.  Right: gated linear attention
  (parts/linear_attention.py);
* ``loop``: layers start .. stop - 1 run `times` times in a row with the same weights, every pass
  with caches and states of its own (a cache slot per (pass, layer) in the schedule); before a
  pass's first layer, row t of ``loop.step`` is added to the residual sum.

Tensor names: ``embed``, ``loop.step``, ``l<i>.norm1|norm1b|norm2|norm2b``, ``l<i>.mix.{q,k,o,q.norm,k.norm}``
or ``l<i>.mix.left.{q,k,v,o,q.norm,k.norm,q.conv,k.conv,v.conv,out}`` and
``l<i>.mix.right.{q,k,v,g,o,norm,a1,a2,a2.b,out}``, ``l<i>.mlp.{up,down}``, ``final.norm``.
"""
from __future__ import annotations

from ..cache.spec import WINDOW_CHUNK, WINDOW_NONE
from ..config.pazatar import DEFAULT_DECAY_RANK, PazatarConfig, SoftmaxMixerConfig
from ..parts.attention import Attention
from ..parts.block import SandwichBlock
from ..parts.feedforward import DenseMLP
from ..parts.linear_attention import GatedLinearAttention
from ..parts.model import DecoderModel, Run
from ..parts.norm import RMSNorm
from ..parts.parallel import ParallelMixers
from ..parts.position import Rotary, WavelengthScaling, YarnRotary, YarnScaling
from ..registry import register_architecture

BLOCK_NAMES = {"norm1": "norm1", "mixer": "mix.", "norm1b": "norm1b", "norm2": "norm2", "ffn": "mlp.", "norm2b": "norm2b"}
ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm",
                   "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv"}
LOOP_TABLE = "loop.step"


def _rotary(m: SoftmaxMixerConfig, left: bool):
    if m.rot is None:
        return None
    sc = m.rot.scaling_dict()
    if left:
        scaling = None if sc is None else WavelengthScaling(sc["factor"], sc["low"], sc["high"], sc["original"])
        return Rotary(m.dim, m.rot.base, scaling, "half", m.rot.dims)
    if sc is None:
        return Rotary(m.dim, m.rot.base, None, "interleaved", m.rot.dims)
    return YarnRotary(m.dim, m.rot.base, YarnScaling(sc["factor"], sc["original"], sc["fast"], sc["slow"]), "interleaved", m.rot.dims)


def _attention(cfg: PazatarConfig, m: SoftmaxMixerConfig, left: bool) -> Attention:
    window = dict(window_kind=WINDOW_CHUNK, window=m.mask_size) if m.mask_size else dict(window_kind=WINDOW_NONE)
    if left:
        return Attention(cfg.width, m.heads, m.kv_heads, m.dim, rotary=_rotary(m, True), qk_norm_eps=cfg.norm_eps,
                         scale=m.scale, v_head_dim=m.vdim, qk_norm_weights="head", conv_taps=m.conv, softcap=m.softcap,
                         sink=True, names=ATTENTION_NAMES, **window)
    return Attention(cfg.width, m.heads, m.kv_heads, m.dim, rotary=_rotary(m, False), qk_norm_eps=cfg.norm_eps,
                     scale=m.scale, qk_norm_weights="projection", values_from_keys=True, names=ATTENTION_NAMES, **window)


def build_pazatar(cfg: PazatarConfig) -> DecoderModel:
    cfg.validate()
    blocks = []
    for layer in cfg.layers:
        if layer.type == "attention":
            mixer = _attention(cfg, layer.attention, left=False)
        else:
            r = layer.linear
            right = GatedLinearAttention(cfg.width, r.heads, r.dim, r.vdim, r.tau, r.decay_rank or DEFAULT_DECAY_RANK, cfg.norm_eps)
            mixer = ParallelMixers(cfg.width, [("left", _attention(cfg, layer.attention, left=True)), ("right", right)], cfg.norm_eps)

        def norm():
            return RMSNorm(cfg.width, cfg.norm_eps, name="")

        ffn = DenseMLP(cfg.width, layer.ff, "relu2", names={"up": "up", "down": "down"}) if layer.ff else None
        blocks.append(SandwichBlock(norm(), mixer, norm(), norm() if ffn else None, ffn, norm() if ffn else None, names=BLOCK_NAMES))
    # the order of the runs: every (pass, layer) of the repeated stretch has a cache slot of its own
    schedule, slot = [], 0
    n = len(cfg.layers)
    order = [(i, None) for i in range(n)]
    if cfg.has_loop:
        order = [(i, None) for i in range(cfg.loop_start)]
        for t in range(cfg.loop_times):
            order += [(i, t) for i in range(cfg.loop_start, cfg.loop_stop)]
        order += [(i, None) for i in range(cfg.loop_stop, n)]
    for i, t in order:
        first_of_pass = t is not None and i == cfg.loop_start
        schedule.append(Run(i, slot, add_row=(LOOP_TABLE, t) if first_of_pass else None))
        slot += 1
    return DecoderModel(cfg.vocab_size, cfg.width, blocks, RMSNorm(cfg.width, cfg.norm_eps, name=""), schedule=schedule,
                        tie_embeddings=True, config=cfg, layer_prefix="l", embed_name="embed", norm_prefix="final.norm",
                        row_tables={LOOP_TABLE: cfg.loop_times} if cfg.has_loop else None)


register_architecture("Pazatar", PazatarConfig, build_pazatar)
