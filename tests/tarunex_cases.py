"""Small Tarunex configurations and helpers shared by the CPU and GPU tests of that design."""
import copy
import json
import os

import torch
from safetensors.torch import load_file, save_file

from tests.plain.tarunex_plain import PlainTarunex


def _attention(heads, kv_heads, dim, vdim, scale, softcap, coef, every):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, softcap=softcap, q_temp=dict(coef=coef, every=every))


def _latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, base=10000.0, dims=None):
    return dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, q_rank=q_rank, scale=scale,
                rot=dict(base=base, dims=rot_dim if dims is None else dims))


def _moe(ff, experts, top, shared):
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top), shared=dict(ff=shared))


def _layer(kind, mixer, mlp=None):
    return dict(type=kind, mixer=mixer, mlp=mlp)


#: every size differs from every other: value heads larger and smaller than key heads, fewer kv heads than heads, a layer
#: without a feed-forward, a loop in the middle that holds both kinds of mixer and is walked three times, a temperature
#: that steps every five positions
TAR_A = dict(architecture="Tarunex", vocab=89, width=40, norm=dict(eps=2e-6), embedding=dict(scale=3.0), logit_scale=0.7, logit_softcap=12.0,
             loop=dict(start=1, stop=3, times=3),
             layers=[_layer("latent_attention", _latent(3, 5, 6, 7, 9, 11, 0.25, base=500.0), _moe(12, 6, 2, 10)),
                     _layer("attention", _attention(4, 2, 6, 10, 0.3, 5.0, 0.4, 5), _moe(20, 8, 3, 14)),
                     _layer("latent_attention", _latent(2, 7, 4, 3, 6, 5, 0.4), _moe(8, 5, 1, 6)),
                     _layer("attention", _attention(3, 3, 8, 4, 0.2, 9.0, 0.15, 3)),
                     _layer("attention", _attention(2, 1, 4, 4, 0.5, 2.5, 0.8, 16), _moe(16, 4, 4, 4))])

#: values that may happen to be equal or 1 elsewhere: one head, one expert of one, a loop of one walk over all layers, a
#: temperature that steps at every position, no scaling of embedding and logits, equal sizes
TAR_B = dict(architecture="Tarunex", vocab=61, width=32, norm=dict(eps=1e-5), embedding=dict(scale=1.0), logit_scale=1.0, logit_softcap=18.0,
             loop=dict(start=0, stop=3, times=1),
             layers=[_layer("attention", _attention(1, 1, 8, 8, 1.0, 24.0, 0.35, 1), _moe(32, 1, 1, 32)),
                     _layer("latent_attention", _latent(1, 8, 8, 8, 8, 8, 0.25), _moe(8, 4, 4, 8)),
                     _layer("attention", _attention(4, 4, 8, 8, 0.35, 1.0, 1.0, 2), _moe(8, 4, 1, 8))])

#: no loop at all, the latent attention first and last
TAR_PLAIN = dict(architecture="Tarunex", vocab=53, width=24, norm=dict(eps=1e-6), embedding=dict(scale=5.0), logit_scale=2.0, logit_softcap=8.0,
                 layers=[_layer("latent_attention", _latent(2, 4, 4, 6, 5, 7, 0.3, base=100.0, dims=2), _moe(8, 3, 2, 12)),
                         _layer("attention", _attention(2, 1, 6, 5, 0.4, 4.0, 0.25, 4), _moe(10, 4, 2, 6)),
                         _layer("latent_attention", _latent(3, 2, 6, 4, 8, 3, 0.35))])

#: the loop at the end and over one layer, walked four times
TAR_TAIL = dict(architecture="Tarunex", vocab=47, width=28, norm=dict(eps=3e-6), embedding=dict(scale=2.0), logit_scale=0.5, logit_softcap=20.0,
                loop=dict(start=1, stop=2, times=4),
                layers=[_layer("attention", _attention(2, 2, 5, 7, 0.4, 6.0, 0.2, 7), _moe(9, 3, 2, 5)),
                        _layer("latent_attention", _latent(2, 3, 4, 5, 7, 6, 0.3), _moe(7, 5, 2, 11))])

#: the loop from the first layer on, its last layer without a feed-forward: a walk's start meets a single pending addend
TAR_BARE = dict(architecture="Tarunex", vocab=59, width=36, norm=dict(eps=2e-6), embedding=dict(scale=1.5), logit_scale=1.25, logit_softcap=40.0,
                loop=dict(start=0, stop=2, times=3),
                layers=[_layer("latent_attention", _latent(2, 6, 2, 5, 4, 7, 0.3, base=50.0), _moe(6, 3, 2, 9)),
                        _layer("attention", _attention(6, 2, 3, 5, 0.45, 7.0, 0.5, 9)),
                        _layer("attention", _attention(2, 2, 7, 3, 0.3, 3.5, 0.1, 2), _moe(5, 2, 1, 7))])

#: sizes that the products' tiled kernels and the MFMA attention, latent attention and expert kernels take in bfloat16
TAR_C = dict(architecture="Tarunex", vocab=400, width=128, norm=dict(eps=4e-6), embedding=dict(scale=8.0), logit_scale=0.5, logit_softcap=25.0,
             loop=dict(start=0, stop=2, times=2),
             layers=[_layer("attention", _attention(4, 2, 64, 32, 0.12, 20.0, 0.25, 32), _moe(64, 8, 2, 64)),
                     _layer("latent_attention", _latent(4, 32, 16, 32, 64, 48, 0.14), _moe(128, 4, 1, 32)),
                     _layer("attention", _attention(8, 2, 32, 48, 0.18, 10.0, 0.2, 64), _moe(64, 16, 4, 128))])

#: one attention layer and one latent layer: far keys among hundreds
TAR_FAR = dict(architecture="Tarunex", vocab=83, width=48, norm=dict(eps=1e-6), embedding=dict(scale=4.0), logit_scale=0.8, logit_softcap=15.0,
               loop=dict(start=0, stop=2, times=2),
               layers=[_layer("attention", _attention(3, 1, 16, 16, 0.25, 25.0, 0.45, 100), _moe(24, 4, 2, 16)),
                       _layer("latent_attention", _latent(3, 8, 8, 8, 16, 12, 0.25, base=100000.0), _moe(16, 4, 2, 8))])

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
    """Queries scaled so that a softmax has few large terms: a key that is missed or wrongly seen changes the result by
    much more than rounding, also among hundreds of keys; the penalty on the distance made small, so that far keys keep
    their weight."""
    def tweak(tensors):
        for name in tensors:
            if name.endswith(".mix.q") or name.endswith(".mix.uq"):
                tensors[name] = (tensors[name].float() * factor).to(tensors[name].dtype)
            if name.endswith(".mix.r1"):
                tensors[name] = (tensors[name].float() * 0.1).to(tensors[name].dtype)
    return tweak


def heavy_sink(shift=-4.0):
    """Attention scores pushed down (key biases against the query biases), so that the one in the softmax's denominator
    takes a large share: a sink that is left out or counted twice shows."""
    def tweak(tensors):
        for name in list(tensors):
            if name.endswith(".mix.q.b"):
                tensors[name] = torch.full_like(tensors[name], 1.0)
                k = name[:-len("q.b")] + "k.b"
                tensors[k] = torch.full_like(tensors[k], shift)
    return tweak


def strong_penalty(r1=1.5, r2=3.0):
    """A penalty on the distance that decides which keys weigh: a distance that is one off shows."""
    def tweak(tensors):
        for name in tensors:
            if name.endswith(".mix.r1"):
                tensors[name] = torch.full_like(tensors[name], r1)
            if name.endswith(".mix.r2"):
                tensors[name] = torch.full_like(tensors[name], r2)
    return tweak


def decisive_router(factor=4.0):
    """Router logits spread out, so that fewer choices hang on a difference of the size of a bfloat16 rounding."""
    def tweak(tensors):
        for name in tensors:
            if name.endswith(".mlp.router") or name.endswith(".mlp.router.b"):
                tensors[name] = (tensors[name].float() * factor).to(tensors[name].dtype)
    return tweak


def both(*tweaks):
    def tweak(tensors):
        for t in tweaks:
            t(tensors)
    return tweak


def plain_logits(folder, requests):
    plain = PlainTarunex.from_folder(folder)
    return {rid: plain.forward(toks) for rid, toks in requests.items()}


def vocab_of(folder):
    with open(os.path.join(folder, "config.json")) as f:
        return json.load(f)["vocab"]
