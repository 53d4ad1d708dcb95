"""Kuvonex: a decoder of latent attention layers with routed feed-forwards and norms on the
branches' outputs, assembled from config.json layer by layer.

* embedding rows times ``embedding.scale``;
* every layer x += norm1(mixer(x)), then x += norm2(ff(x)) where it has a feed-forward;
* the mixer attends over one latent row per token (parts/latent_attention.py), with a sink in the
  softmax and a sigmoid gate on the heads' outputs; a layer with ``kv_from`` keeps no latent of
  its own and reads the cache of the layer it names (an entry of the schedule with write=False);
* the feed-forward is a mixture of SiLU-gated experts: sigmoid router in float, experts chosen by
  score + correction among the best groups, outputs weighted by the uncorrected scores;
* final norm and head.

Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.{q,dkv,dkv.norm,uk,uv,sink,g,o}``,
``l<i>.mlp.{router,correction,e<j>.gate,e<j>.up,e<j>.down}``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config.kuvonex import KuvonexConfig
from ..parts.block import PostNormBlock
from ..parts.feedforward import MoESwiGLU
from ..parts.latent_attention import LatentAttention
from ..parts.model import DecoderModel, Run
from ..parts.norm import RMSNorm
from ..parts.position import Rotary
from ..registry import register_architecture

BLOCK_NAMES = {"norm1": "norm1", "mixer": "mix.", "norm2": "norm2", "ffn": "mlp."}
MLP_NAMES = {"router": "router", "correction": "correction", "gate": "e{e}.gate", "up": "e{e}.up", "down": "e{e}.down"}


def build_kuvonex(cfg: KuvonexConfig) -> DecoderModel:
    cfg.validate()
    blocks, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        rotary = Rotary(m.rot_dim, m.rot_base, None, "interleaved", m.rot_dims)
        mixer = LatentAttention(cfg.width, m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, rotary, cfg.norm_eps, m.scale,
                                sink=True, gate=True, own_latent=m.kv_from is None)
        ffn = norm2 = None
        if layer.mlp is not None:
            f = layer.mlp
            ffn = MoESwiGLU(cfg.width, f.experts, f.top, f.ff, shared_intermediate=None, gate="sigmoid", renormalise=False,
                            score_on_input=False, activation="silu", correction=True, n_groups=f.groups,
                            keep_groups=f.keep, names=MLP_NAMES)
            norm2 = RMSNorm(cfg.width, cfg.norm_eps, name="")
        blocks.append(PostNormBlock(RMSNorm(cfg.width, cfg.norm_eps, name=""), mixer, norm2, ffn, names=BLOCK_NAMES))
        schedule.append(Run(i, i) if m.kv_from is None else Run(i, m.kv_from, write=False))
    return DecoderModel(cfg.vocab_size, cfg.width, blocks, RMSNorm(cfg.width, cfg.norm_eps, name=""), schedule=schedule,
                        tie_embeddings=False, config=cfg, layer_prefix="l", embed_name="embed", norm_prefix="final.norm",
                        head_name="head", embedding_scale=cfg.embedding_scale)


register_architecture("Kuvonex", KuvonexConfig, build_kuvonex)
