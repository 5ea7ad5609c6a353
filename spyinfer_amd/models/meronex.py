"""Meronex from parts: a plain embedding and an output head of its own, pre-norm blocks whose norms work on groups of
the vector and whose sublayers' results pass a sigmoid gate and a constant, mixers 'mlstm', 'delta' and 'parallel' (an
attention beside a time mix) in the order the configuration lists, mixtures of experts as feed-forwards, a final norm of
the same kind.  Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.mix.*``, ``l<i>.rg1``, ``l<i>.norm2``, ``l<i>.mlp.*``,
``l<i>.rg2``, ``final.norm``, ``head``."""
from __future__ import annotations

from ..config.model_config import MeronexConfig
from ..config.registry import register_architecture
from ..parts import (HeadDelta, LMHead, MLSTM, MoEMLP, PagedAttention, PreNormBlock, ResultGate, RMSNorm, RotaryEmbedding, SideBySide,
                     TimeMix, TokenEmbedding)
from .base import DecoderModel

ATTENTION_NAMES = dict(q=".q", k=".k", v=".v", o=".o")


def build_meronex(cfg: MeronexConfig) -> DecoderModel:
    W, eps, groups, mult = cfg.width, cfg.norm_eps, cfg.norm_groups, cfg.residual_mult

    def norm():
        return RMSNorm(W, eps, suffix="", groups=groups)
    layers = []
    for layer in cfg.layers:
        m = layer["mixer"]
        if layer["type"] == "mlstm":
            mixer = MLSTM(W, m["heads"], m["dim"], m["vdim"], m["gate_cap"], eps)
        elif layer["type"] == "delta":
            mixer = HeadDelta(W, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"], eps)
        else:
            a, t = m["left"], m["right"]
            rot = a["rot"]
            position = RotaryEmbedding(a["dim"], rot["base"], rot["dims"], rot["scaling"]) if rot else None
            left = PagedAttention(W, a["heads"], a["kv_heads"], a["dim"], position, scale=a["scale"], value_dim=a["vdim"],
                                  names=ATTENTION_NAMES, softcap=a["softcap"], value_norm_eps=eps)
            mixer = SideBySide(W, left, TimeMix(W, t["heads"], t["dim"], eps, t["decay_rank"]), eps)
        f = layer["mlp"]
        ffn = None
        if f is not None:
            ffn = MoEMLP(W, f["ff"], f["experts"], f["top"], score="sigmoid", renormalize=False, correction=False, weight_on="input", activation="clamped", limit=f["limit"])
        gates = (ResultGate(W, mult), ResultGate(W, mult) if ffn is not None else None)
        layers.append(PreNormBlock(norm(), mixer, norm() if ffn is not None else None, ffn, names=("norm1", "mix", "norm2", "mlp"), gates=gates))
    names = dict(embed="embed", layers="l%d", final_norm="final.norm", lm_head="head")
    return DecoderModel(cfg, TokenEmbedding(cfg.vocab, W, suffix=""), None, layers, norm(), LMHead(cfg.vocab, W, suffix=""), None, names)


register_architecture("Meronex", MeronexConfig, build_meronex)
