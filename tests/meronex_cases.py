"""Small Meronex configurations and helpers shared by the CPU and GPU tests of that design."""
import copy
import json
import os

import torch
from safetensors.torch import load_file, save_file

from tests.plain.meronex_plain import PlainMeronex


def _left(heads, kv_heads, dim, vdim, scale, softcap=None, base=10000.0, dims=None, scaling=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if softcap is not None:
        m["softcap"] = softcap
    if dims:
        m["rot"] = dict(base=base, dims=dims)
        if scaling:
            m["rot"]["scaling"] = scaling
    return m


def _parallel(left, heads, dim, rank):
    return dict(left=left, right=dict(heads=heads, dim=dim, decay_rank=rank))


def _mlstm(heads, dim, vdim, cap):
    return dict(heads=heads, dim=dim, vdim=vdim, gate_cap=cap)


def _delta(heads, kv_heads, dim, vdim, conv):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv)


def _moe(ff, limit, experts, top):
    return dict(kind="moe", expert=dict(ff=ff, limit=limit), router=dict(experts=experts, top=top))


def _layer(kind, mixer, mlp=None):
    return dict(type=kind, mixer=mixer, mlp=mlp)


RAMP = dict(factor=8.0, original=64, fast=4.0, slow=1.0)

#: every size differs from every other: value heads larger and smaller than key heads, fewer kv heads than heads in the
#: attention and in the delta rule, a layer without a feed-forward, an attention without a cap and without scaling, one
#: without any rotation, several experts chosen, three norm groups
MER_A = dict(architecture="Meronex", vocab=97, width=48, norm=dict(eps=3e-6, groups=3), residual_mult=0.7,
             layers=[_layer("parallel", _parallel(_left(4, 2, 8, 6, 0.3, softcap=4.0, dims=4, scaling=RAMP), 3, 4, 5), _moe(24, 1.5, 8, 3)),
                     _layer("mlstm", _mlstm(3, 5, 7, 10.0), _moe(20, 3.0, 6, 2)),
                     _layer("delta", _delta(4, 2, 6, 5, 3)),
                     _layer("parallel", _parallel(_left(2, 1, 6, 10, 0.25, base=500.0, dims=6), 2, 5, 3), _moe(12, 0.8, 5, 1)),
                     _layer("mlstm", _mlstm(2, 9, 4, 3.0)),
                     _layer("delta", _delta(3, 3, 4, 8, 4), _moe(16, 2.5, 4, 4)),
                     _layer("parallel", _parallel(_left(3, 3, 4, 4, 0.5, softcap=1.5), 1, 6, 2), _moe(8, 1.0, 3, 2))])

#: values that may happen to be equal or 1 elsewhere: one head, one norm group, a multiplier of one, one tap, one expert
#: of one, equal sizes, a recurrence first, a parallel layer last
MER_B = dict(architecture="Meronex", vocab=61, width=32, norm=dict(eps=2e-5, groups=1), residual_mult=1.0,
             layers=[_layer("delta", _delta(1, 1, 8, 8, 1), _moe(32, 1.0, 1, 1)),
                     _layer("parallel", _parallel(_left(1, 1, 8, 8, 1.0, softcap=30.0, dims=8), 1, 8, 8), _moe(32, 4.0, 4, 1)),
                     _layer("mlstm", _mlstm(1, 8, 8, 14.0)),
                     _layer("delta", _delta(2, 1, 8, 8, 2), _moe(8, 2.0, 4, 4)),
                     _layer("parallel", _parallel(_left(4, 4, 8, 8, 0.5, dims=2, scaling=dict(factor=2.0, original=8, fast=2.0, slow=1.0)), 4, 8, 1))])

#: sizes that the products' tiled kernels and the MFMA attention and expert kernels take in bfloat16
MER_C = dict(architecture="Meronex", vocab=400, width=128, norm=dict(eps=4e-6, groups=2), residual_mult=0.6,
             layers=[_layer("mlstm", _mlstm(2, 32, 64, 12.0), _moe(64, 2.0, 8, 2)),
                     _layer("parallel", _parallel(_left(4, 2, 32, 48, 0.18, softcap=20.0, base=100000.0, dims=16,
                                                        scaling=dict(factor=3.0, original=32, fast=8.0, slow=1.0)), 2, 64, 16), _moe(128, 3.0, 4, 1)),
                     _layer("delta", _delta(4, 2, 32, 16, 4), _moe(64, 1.5, 16, 4)),
                     _layer("parallel", _parallel(_left(4, 1, 64, 32, 0.12, softcap=8.0, dims=64), 4, 16, 8))])

#: one parallel layer: far keys, a state that must survive hundreds of tokens
MER_FAR = dict(architecture="Meronex", vocab=83, width=40, norm=dict(eps=1e-6, groups=5), residual_mult=0.9,
               layers=[_layer("parallel", _parallel(_left(3, 1, 12, 10, 0.35, softcap=25.0, base=100000.0, dims=8,
                                                          scaling=dict(factor=4.0, original=256, fast=16.0, slow=1.0)), 2, 6, 4), _moe(24, 2.0, 4, 2))])

#: no parallel layer at all: no page group, only state slots
MER_REC = dict(architecture="Meronex", vocab=53, width=24, norm=dict(eps=1e-5, groups=2), residual_mult=0.5,
               layers=[_layer("mlstm", _mlstm(2, 4, 6, 9.0), _moe(8, 2.0, 4, 2)),
                       _layer("delta", _delta(2, 1, 4, 6, 3), _moe(8, 1.0, 3, 1))])

#: sizes that are multiples of nothing: rows of the products that no vector load fits, heads of odd sizes
MER_ODD = dict(architecture="Meronex", vocab=77, width=50, norm=dict(eps=1e-6, groups=5), residual_mult=0.45,
               layers=[_layer("parallel", _parallel(_left(6, 3, 10, 7, 0.3, softcap=6.0, base=3000.0, dims=6,
                                                          scaling=dict(factor=16.0, original=32, fast=3.0, slow=0.5)), 5, 7, 3), _moe(18, 1.2, 7, 3)),
                       _layer("mlstm", _mlstm(5, 7, 9, 8.0), _moe(11, 2.0, 3, 2)),
                       _layer("delta", _delta(6, 2, 5, 11, 5), _moe(13, 0.7, 9, 1))])

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
            if name.endswith(".mix.left.q"):
                tensors[name] = (tensors[name].float() * factor).to(tensors[name].dtype)
    return tweak


def long_memory(forget_bias=6.0, a_log=-4.0, w0=-5.0):
    """Recurrences that forget slowly: forget gates near one and small decay rates, so that what a state took in
    hundreds of tokens ago still weighs in the output (a lost or restarted state shows)."""
    def tweak(tensors):
        for name in tensors:
            if name.endswith(".mix.f.b"):
                tensors[name] = torch.full_like(tensors[name], forget_bias)
            if name.endswith(".mix.A_log"):
                tensors[name] = torch.full_like(tensors[name], a_log)
            if name.endswith(".mix.right.w0"):
                tensors[name] = torch.full_like(tensors[name], w0)
    return tweak


def decisive_router(factor=4.0):
    """Router logits spread out, so that fewer choices hang on a difference of the size of a bfloat16 rounding."""
    def tweak(tensors):
        for name in tensors:
            if name.endswith(".mlp.router"):
                tensors[name] = (tensors[name].float() * factor).to(tensors[name].dtype)
    return tweak


def both(*tweaks):
    def tweak(tensors):
        for t in tweaks:
            t(tensors)
    return tweak


def plain_logits(folder, requests):
    plain = PlainMeronex.from_folder(folder)
    return {rid: plain.forward(toks) for rid, toks in requests.items()}


def vocab_of(folder):
    with open(os.path.join(folder, "config.json")) as f:
        return json.load(f)["vocab"]
