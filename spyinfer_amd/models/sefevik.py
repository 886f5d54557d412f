"""Sefevik from parts: an embedding with a hashed pair table, blocks that norm a sublayer's output and hand on a learned
mix of all layer results, minGRU and latent-attention mixers in the order the configuration lists, dense feed-forwards
with the xIELU activation, a final RMS norm and an untied head.  Tensor names: ``embed``, ``bigram``, ``l<i>.norm1``,
``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``l<i>.dwa``, ``final.norm``, ``head``."""
from __future__ import annotations

from ..config.model_config import SefevikConfig
from ..config.registry import register_architecture
from ..parts import (DenseMLP, DepthMix, LatentAttention, LMHead, MinGRU, OutputNormBlock, PairHashEmbedding, RMSNorm,
                     RotaryEmbedding)
from .base import DecoderModel, LayerCall


def build_sefevik(cfg: SefevikConfig) -> DecoderModel:
    H, eps, n = cfg.width, cfg.norm_eps, len(cfg.layers)
    embed = PairHashEmbedding(cfg.vocab, H, cfg.bigram_buckets, cfg.bigram_mul_prev, cfg.bigram_mul_cur)
    # a layer that reads another's cache may look further back than that layer itself: the rows are kept for the
    # largest window of their readers (None = for good)
    keep = {}
    for i, layer in enumerate(cfg.layers):
        if layer["type"] == "latent_attention":
            src = layer["mixer"]["kv_from"] if layer["mixer"]["kv_from"] is not None else i
            w = layer["mixer"]["window"]
            keep[src] = None if (w is None or (src in keep and keep[src] is None)) else max(w, keep.get(src, 0))
    layers, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        m = layer["mixer"]
        if layer["type"] == "mingru":
            mixer = MinGRU(H, m["width"])
            schedule.append(LayerCall(i, i))
        else:
            rot = m["rot"]
            position = RotaryEmbedding(m["rot_dim"], rot["base"], rot["dims"], rot["scaling"]) if rot else None
            src = m["kv_from"]
            mixer = LatentAttention(H, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["scale"], eps, position,
                                    window=m["window"], cache_window=keep[i if src is None else src], shares_cache=src is not None)
            schedule.append(LayerCall(i, i, True) if src is None else LayerCall(i, src, False))
        ffn = DenseMLP(H, layer["mlp"]["ff"]) if layer["mlp"] else None
        layers.append(OutputNormBlock(mixer, RMSNorm(H, eps, suffix=""), ffn, RMSNorm(H, eps, suffix="") if ffn else None,
                                      DepthMix(i, n)))
    names = dict(embed="", layers="l%d", final_norm="final.norm", lm_head="head")
    return DecoderModel(cfg, embed, None, layers, RMSNorm(H, eps, suffix=""), LMHead(cfg.vocab, H, suffix=""), schedule, names)


register_architecture("Sefevik", SefevikConfig, build_sefevik)
