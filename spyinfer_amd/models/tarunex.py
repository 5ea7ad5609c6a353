"""Tarunex from parts: a scaled embedding, blocks whose mixer and feed-forward read the stream through a norm each (a
norm's weight is one number) and are added together, mixers 'attention' and 'latent_attention' in the order the
configuration lists, a mixture of gated experts with a router bias and an expert for every token, a run of layers that may
be walked several times with the same weights (every walk with caches of its own), a final norm, a head of its own and
scaled, capped logits.  Tensor names: ``embed``, ``loop.step``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``,
``l<i>.mlp.*``, ``final.norm``, ``head``."""
from __future__ import annotations

from ..config.model_config import TarunexConfig
from ..config.registry import register_architecture
from ..parts import (GatedMLP, LatentAttention, LMHead, MoEMLP, PagedAttention, ParallelBlock, PassEntry, RMSNorm, RotaryEmbedding,
                     TokenEmbedding)
from .base import DecoderModel, LayerCall

ATTENTION_NAMES = dict(q=".q", k=".k", v=".v", o=".o", g=".g", bias=".b", r1=".r1", r2=".r2")
FF_NAMES = (".gate", ".up", ".down")


def run_order(n_layers: int, loop):
    """The calls of a forward pass: the layers of ``loop`` (start .. stop - 1) walked ``times`` times in a row, every walk
    with cache ids of its own and its first call marked as the walk's start; the other layers once."""
    if not loop:
        return [LayerCall(i, i) for i in range(n_layers)]
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    calls = [LayerCall(i, i) for i in range(start)]
    for walk in range(times):
        for i in range(start, stop):
            calls.append(LayerCall(i, len(calls), True, walk if i == start else None))
    for i in range(stop, n_layers):
        calls.append(LayerCall(i, len(calls)))
    return calls


def build_tarunex(cfg: TarunexConfig) -> DecoderModel:
    W, eps = cfg.width, cfg.norm_eps
    embed = TokenEmbedding(cfg.vocab, W, scale=cfg.embedding_scale, suffix="")
    layers = []
    for layer in cfg.layers:
        m = layer["mixer"]
        if layer["type"] == "attention":
            temp = (m["q_temp"]["coef"], m["q_temp"]["every"]) if m["q_temp"] else None
            mixer = PagedAttention(W, m["heads"], m["kv_heads"], m["dim"], None, scale=m["scale"], value_dim=m["vdim"], bias=True,
                                   gate="head", names=ATTENTION_NAMES, softcap=m["softcap"], query_temperature=temp,
                                   distance_penalty=True, zero_sink=True)
        else:
            rot = m["rot"]
            position = RotaryEmbedding(m["rot_dim"], rot["base"], rot["dims"], interleaved=True) if rot else None
            mixer = LatentAttention(W, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["scale"], eps, position,
                                    window=None, sink=False, q_rank=m["q_rank"], gate=True)
        f = layer["mlp"]
        ffn = None
        if f is not None:
            shared = GatedMLP(W, f["shared_ff"], names=FF_NAMES) if f["shared_ff"] else None
            ffn = MoEMLP(W, f["ff"], f["experts"], f["top"], correction=False, router_bias=True, shared=shared)
        layers.append(ParallelBlock(RMSNorm(W, eps, suffix="", scalar=True), mixer, ffn,
                                    norm2=RMSNorm(W, eps, suffix="", scalar=True) if ffn is not None else None))
    names = dict(embed="embed", layers="l%d", final_norm="final.norm", lm_head="head", pass_entry="loop.step")
    entry = PassEntry(W, cfg.loop["times"]) if cfg.loop else None
    return DecoderModel(cfg, embed, None, layers, RMSNorm(W, eps, suffix="", scalar=True),
                        LMHead(cfg.vocab, W, suffix="", scale=cfg.logit_scale, softcap=cfg.logit_softcap),
                        run_order(len(layers), cfg.loop), names, pass_entry=entry)


register_architecture("Tarunex", TarunexConfig, build_tarunex)
