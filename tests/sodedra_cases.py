"""Small Sodedra configurations and helpers shared by the CPU and GPU tests of that design."""
import copy
import json
import os

import torch
from safetensors.torch import load_file, save_file

from tests.plain.sodedra_plain import PlainSodedra


def _attention(heads, kv_heads, dim, vdim, scale, window=None, base=10000.0, dims=None, scaling=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if dims:
        m["rot"] = dict(base=base, dims=dims)
        if scaling:
            m["rot"]["scaling"] = scaling
    if window is not None:
        m["mask"] = dict(size=window)
    return m


def _mlstm(heads, dim, vdim, cap):
    return dict(heads=heads, dim=dim, vdim=vdim, gate_cap=cap)


def _delta(heads, kv_heads, dim, vdim, conv, decay_rank, gate_rank):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv, decay_rank=decay_rank, gate_rank=gate_rank)


def _dense(ff):
    return dict(kind="dense", ff=ff)


def _moe(ff, experts, top, groups, keep, scale):
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top, scale=scale, groups=dict(count=groups, keep=keep)))


def _layer(kind, mixer, mlp=None):
    return dict(type=kind, mixer=mixer, mlp=mlp)


WAVE = dict(factor=8.0, low=1.0, high=4.0, original=64)

#: every size differs from every other: value heads larger and smaller than key heads, fewer kv heads than heads in the
#: attention and in the delta rule, a layer without a feed-forward, an attention without window and without scaling, one
#: without any rotation, mixtures with several groups
SOD_A = dict(architecture="Sodedra", vocab=97, width=48, norm=dict(eps=3e-6), embedding=dict(scale=0.7),
             layers=[_layer("attention", _attention(4, 2, 8, 6, 0.3, window=9, dims=4, scaling=WAVE), _moe(24, 8, 3, 4, 2, 1.3)),
                     _layer("mlstm", _mlstm(3, 5, 7, 10.0), _dense(72)),
                     _layer("channel_delta", _delta(4, 2, 6, 5, 3, 7, 5)),
                     _layer("attention", _attention(2, 1, 6, 10, 0.25, base=500.0, dims=6), _dense(56)),
                     _layer("mlstm", _mlstm(2, 9, 4, 3.0), _moe(20, 6, 2, 3, 2, 0.8)),
                     _layer("channel_delta", _delta(3, 3, 4, 8, 4, 3, 6), _dense(40)),
                     _layer("attention", _attention(3, 3, 4, 4, 0.5, window=5), _dense(32))])

#: values that may happen to be equal or 1 elsewhere: one head, windows of one and two tokens, one tap, one expert chosen
#: of one group, equal sizes, a recurrence first, an embedding scale of one
SOD_B = dict(architecture="Sodedra", vocab=61, width=32, norm=dict(eps=2e-5), embedding=dict(scale=1.0),
             layers=[_layer("channel_delta", _delta(1, 1, 8, 8, 1, 4, 4), _dense(32)),
                     _layer("attention", _attention(1, 1, 8, 8, 1.0, window=1, dims=8), _moe(32, 4, 1, 1, 1, 1.0)),
                     _layer("mlstm", _mlstm(1, 8, 8, 14.0)),
                     _layer("attention", _attention(4, 4, 8, 8, 0.5, window=2, dims=2, scaling=dict(factor=2.0, low=1.0, high=1.0, original=8)), _dense(32)),
                     _layer("channel_delta", _delta(2, 1, 8, 8, 2, 1, 1), _moe(8, 4, 4, 2, 2, 2.0))])

#: sizes that the products' tiled kernels and the MFMA attention take in bfloat16
SOD_C = dict(architecture="Sodedra", vocab=400, width=128, norm=dict(eps=4e-6), embedding=dict(scale=0.5),
             layers=[_layer("mlstm", _mlstm(2, 32, 64, 12.0), _dense(256)),
                     _layer("attention", _attention(4, 2, 32, 32, 0.18, window=24, base=100000.0, dims=16,
                                                    scaling=dict(factor=3.0, low=1.0, high=3.0, original=32)), _moe(64, 8, 2, 4, 2, 1.5)),
                     _layer("channel_delta", _delta(4, 2, 32, 16, 4, 16, 16), _dense(128)),
                     _layer("attention", _attention(4, 1, 16, 48, 0.2, window=70, dims=8), _dense(256))])

#: one attention layer that sees everything: far keys
SOD_FAR = dict(architecture="Sodedra", vocab=83, width=40, norm=dict(eps=1e-6), embedding=dict(scale=1.5),
               layers=[_layer("attention", _attention(3, 1, 12, 10, 0.35, base=100000.0, dims=8, scaling=dict(factor=4.0, low=1.0, high=4.0, original=256)),
                              _dense(48))])

#: windows of hundreds of tokens over long requests, recurrences between them
SOD_LONG = dict(architecture="Sodedra", vocab=211, width=64, norm=dict(eps=1e-6), embedding=dict(scale=0.9),
                layers=[_layer("attention", _attention(4, 2, 16, 16, 0.3, window=333, base=50000.0, dims=12,
                                                       scaling=dict(factor=6.0, low=1.0, high=5.0, original=512)), _dense(96)),
                        _layer("mlstm", _mlstm(2, 16, 24, 13.0), _moe(32, 6, 2, 3, 2, 1.2)),
                        _layer("channel_delta", _delta(2, 1, 16, 24, 4, 8, 8)),
                        _layer("attention", _attention(2, 2, 8, 24, 0.4, window=150, base=50000.0, dims=8), _dense(64))])

#: no attention layer at all: no page group, only state slots
SOD_REC = dict(architecture="Sodedra", vocab=53, width=24, norm=dict(eps=1e-5), embedding=dict(scale=1.2),
               layers=[_layer("mlstm", _mlstm(2, 4, 6, 9.0), _dense(32)),
                       _layer("channel_delta", _delta(2, 1, 4, 6, 3, 3, 3), _moe(8, 4, 2, 2, 1, 1.1))])

INIT = dict(matrix_std=0.12, norm_std=0.2, bias_std=0.3)


def write_model(folder, config, seed, tweak=None, dtype=torch.bfloat16):
    """A model folder with random weights; ``tweak(tensors)`` may change them before they are written."""
    from spyinfer_amd.weights import write_random_model
    write_random_model(folder, copy.deepcopy(config), seed, dtype, **INIT)
    if tweak is not None:
        path = os.path.join(folder, "model.safetensors")
        tensors = load_file(path)
        tweak(tensors)
        save_file({k: v.contiguous() for k, v in tensors.items()}, path)
    return folder


def sharpen(factor=6.0):
    """Queries scaled so that a softmax has few large terms: a key that is missed or wrongly seen changes the result
    by much more than rounding, also among hundreds of keys."""
    def tweak(tensors):
        for name in tensors:
            if name.endswith(".mix.q") and (name[:-1] + "q.b") in tensors:
                tensors[name] = (tensors[name].float() * factor).to(tensors[name].dtype)
    return tweak


def long_memory(forget_bias=6.0, a_log=-4.0):
    """Recurrences that forget slowly: forget gates near one and small decay rates, so that what the state took in
    hundreds of tokens ago still weighs in the output (a lost or restarted state shows)."""
    def tweak(tensors):
        for name in tensors:
            if name.endswith(".mix.f.b"):
                tensors[name] = torch.full_like(tensors[name], forget_bias)
            if name.endswith(".mix.A_log"):
                tensors[name] = torch.full_like(tensors[name], a_log)
    return tweak


def biased_router(value=0.4):
    """Corrections large enough to change which experts are chosen (they must not enter the weights)."""
    def tweak(tensors):
        for name in tensors:
            if name.endswith(".mlp.correction"):
                t = tensors[name].float()
                t[::2] += value
                t[1::2] -= value
                tensors[name] = t.to(tensors[name].dtype)
    return tweak


def plain_logits(folder, requests):
    plain = PlainSodedra.from_folder(folder)
    return {rid: plain.forward(toks) for rid, toks in requests.items()}


def vocab_of(folder):
    with open(os.path.join(folder, "config.json")) as f:
        return json.load(f)["vocab"]
