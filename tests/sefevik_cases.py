"""Small Sefevik configurations and helpers shared by the CPU and GPU tests of that design."""
import copy
import json
import os

import torch
from safetensors.torch import load_file, save_file

from tests.plain.sefevik_plain import PlainSefevik


def _latent(heads, dim, rot_dim, vdim, kv_rank, scale, window=None, kv_from=None, base=10000.0, dims=None, scaling=None):
    m = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, scale=scale,
             rot=dict(base=base, dims=rot_dim if dims is None else dims))
    if scaling:
        m["rot"]["scaling"] = scaling
    if window is not None:
        m["mask"] = dict(size=window)
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _layer(kind, mixer, ff=None):
    return dict(type=kind, mixer=mixer, mlp=dict(kind="dense", ff=ff) if ff else None)


YARN = dict(factor=8.0, original=64, fast=16.0, slow=2.0)

#: every size differs from every other; a reader of layer 0's rows with a LARGER window than layer 0 itself; a layer
#: without a feed-forward; a latent layer without a window and without scaling in a page group of its own; rotated
#: dims fewer than the rotated part
SEF_A = dict(architecture="Sefevik", vocab=97, width=48, norm=dict(eps=3e-6),
             embedding=dict(bigram=dict(buckets=53, mul_prev=5, mul_cur=11)),
             layers=[_layer("latent_attention", _latent(3, 8, 4, 6, 20, 0.3, window=9, scaling=YARN), ff=72),
                     _layer("mingru", dict(width=40)),
                     _layer("latent_attention", _latent(5, 6, 4, 10, 20, 0.2, window=13, kv_from=0, scaling=YARN), ff=56),
                     _layer("latent_attention", _latent(2, 12, 8, 14, 28, 0.25, base=500.0, dims=6), ff=64),
                     _layer("mingru", dict(width=24), ff=80)])

#: values that may happen to be equal or 1 elsewhere: one head, a window of one and of two tokens, equal sizes, a
#: recurrence first, no pair table
SEF_B = dict(architecture="Sefevik", vocab=61, width=32, norm=dict(eps=2e-5),
             layers=[_layer("mingru", dict(width=32), ff=32),
                     _layer("latent_attention", _latent(1, 8, 8, 8, 8, 1.0, window=1), ff=40),
                     _layer("latent_attention", _latent(4, 8, 8, 8, 16, 0.5, window=2))])

#: sizes that the products' tiled kernels take in bfloat16 (inner sizes in multiples of 128, outer ones of 16)
SEF_C = dict(architecture="Sefevik", vocab=400, width=128, norm=dict(eps=4e-6),
             embedding=dict(bigram=dict(buckets=211, mul_prev=29, mul_cur=3)),
             layers=[_layer("latent_attention", _latent(4, 32, 16, 32, 112, 0.15, window=24, scaling=dict(factor=3.0, original=32, fast=8.0, slow=1.5)), ff=256),
                     _layer("mingru", dict(width=128), ff=128),
                     _layer("latent_attention", _latent(4, 16, 16, 48, 112, 0.2, window=70, kv_from=0,
                                                        scaling=dict(factor=3.0, original=32, fast=8.0, slow=1.5)), ff=256)])

#: one attention layer that sees everything: far keys
SEF_FAR = dict(architecture="Sefevik", vocab=83, width=40, norm=dict(eps=1e-6),
               embedding=dict(bigram=dict(buckets=29, mul_prev=3, mul_cur=13)),
               layers=[_layer("latent_attention", _latent(3, 12, 8, 10, 24, 0.35, base=100000.0), ff=48)])

#: windows of hundreds of tokens over long requests, a reader with a shorter window than the rows' owner, rows of the
#: width that the MFMA attention takes in its largest form's neighbourhood
SEF_LONG = dict(architecture="Sefevik", vocab=211, width=64, norm=dict(eps=1e-6),
                embedding=dict(bigram=dict(buckets=97, mul_prev=17, mul_cur=5)),
                layers=[_layer("latent_attention", _latent(4, 16, 16, 16, 160, 0.3, window=333, base=50000.0,
                                                           scaling=dict(factor=6.0, original=512, fast=24.0, slow=2.0)), ff=96),
                        _layer("mingru", dict(width=48), ff=64),
                        _layer("latent_attention", _latent(2, 8, 16, 24, 160, 0.4, window=150, kv_from=0, base=50000.0,
                                                           scaling=dict(factor=6.0, original=512, fast=24.0, slow=2.0)))])

INIT = dict(matrix_std=0.12, norm_std=0.2, bias_std=0.7)


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
            if name.endswith(".mix.q"):
                tensors[name] = (tensors[name].float() * factor).to(tensors[name].dtype)
    return tweak


def heavy_sinks(value=3.0):
    """Sinks that take most of every softmax's weight: a sink left out, counted twice or scaled changes every attention
    output by a large factor."""
    def tweak(tensors):
        for name in tensors:
            if name.endswith(".mix.sink"):
                tensors[name] = (tensors[name].float() * 0.3 + value).to(tensors[name].dtype)
    return tweak


def plain_logits(folder, requests):
    plain = PlainSefevik.from_folder(folder)
    return {rid: plain.forward(toks) for rid, toks in requests.items()}


def vocab_of(folder):
    with open(os.path.join(folder, "config.json")) as f:
        return json.load(f)["vocab"]
