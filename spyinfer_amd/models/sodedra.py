"""Sodedra from parts: a scaled embedding whose table is also the output head, blocks whose mixer and feed-forward read
one norm (weights stored around zero) and are added together, mixers 'mlstm', 'attention' and 'channel_delta' in the order
the configuration lists, gated feed-forwards, dense or as a mixture of experts, a final norm of the same kind.  Tensor
names: ``embed``, ``l<i>.norm1``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``."""
from __future__ import annotations

from ..config.model_config import SodedraConfig
from ..config.registry import register_architecture
from ..parts import (ChannelDelta, GatedMLP, LMHead, MLSTM, MoEMLP, PagedAttention, ParallelBlock, RMSNorm, RotaryEmbedding,
                     TokenEmbedding)
from .base import DecoderModel

ATTENTION_NAMES = dict(q=".q", k=".k", v=".v", o=".o", g=".g", bias=".b")


def build_sodedra(cfg: SodedraConfig) -> DecoderModel:
    W, eps = cfg.width, cfg.norm_eps
    embed = TokenEmbedding(cfg.vocab, W, scale=cfg.embedding_scale, suffix="")
    layers = []
    for layer in cfg.layers:
        m = layer["mixer"]
        if layer["type"] == "mlstm":
            mixer = MLSTM(W, m["heads"], m["dim"], m["vdim"], m["gate_cap"], eps)
        elif layer["type"] == "attention":
            rot = m["rot"]
            position = RotaryEmbedding(m["dim"], rot["base"], rot["dims"], rot["scaling"]) if rot else None
            mixer = PagedAttention(W, m["heads"], m["kv_heads"], m["dim"], position, window=m["window"], scale=m["scale"],
                                   value_dim=m["vdim"], bias=True, gate=True, names=ATTENTION_NAMES)
        else:
            mixer = ChannelDelta(W, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"], eps, m["decay_rank"], m["gate_rank"])
        f = layer["mlp"]
        if f is None:
            ffn = None
        elif f["kind"] == "dense":
            ffn = GatedMLP(W, f["ff"], names=(".gate", ".up", ".down"))
        else:
            ffn = MoEMLP(W, f["ff"], f["experts"], f["top"], f["groups"], f["keep"], f["scale"])
        layers.append(ParallelBlock(RMSNorm(W, eps, suffix="", offset=1.0), mixer, ffn))
    names = dict(embed="embed", layers="l%d", final_norm="final.norm", lm_head="head")
    return DecoderModel(cfg, embed, None, layers, RMSNorm(W, eps, suffix="", offset=1.0), LMHead(cfg.vocab, W, tied_to=embed, suffix=""),
                        None, names)


register_architecture("Sodedra", SodedraConfig, build_sodedra)
