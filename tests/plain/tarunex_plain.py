"""Plain, slow Tarunex forward pass: whole sequences, no cache, one function per mechanism.

Tarunex is a decoder whose layers read the stream through TWO norms, one per sublayer, and add
both results at once (``x + mixer(n1(x)) + ff(n2(x))``); a norm's weight is one number.  A run of
consecutive layers may be walked several times with the same weights; every walk but the first
starts by adding the embedding output back, and every walk starts by adding a learned vector of
its own.  A layer's token mixer is one of two: an attention without rotation whose scores are
capped, lowered by a logarithmic penalty on the distance and normalised with a one in the
denominator, with queries that grow with the logarithm of the position; or a latent attention
whose queries also pass through a normed low-rank vector, with interleaved rotary pairs.  Both
multiply every head's result by one sigmoid number.  The feed-forward is a mixture of gated
experts (the weights a softmax over the chosen logits, the router with a bias) plus an expert
that every token uses.  The logits are scaled and capped.

This file shares no code with the ``spyinfer_amd`` package.  It takes a configuration as a
dictionary and the tensors as a dictionary of CPU tensors, and computes in ``dtype``
(float64 by default).
"""
import json
import math
import os

import torch


# ---- pieces ------------------------------------------------------------------------------
def rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """RMS norm whose weight is a single number."""
    return rms(x, eps) * g


def silu(z):
    return z * torch.sigmoid(z)


def capped(z, cap):
    return cap * torch.tanh(z / cap)


def gated_ff(h, gate, up, down):
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


def route_chosen_softmax(z, top):
    """Router logits z [T, E] -> (chosen experts [T, top], softmax over the chosen logits alone [T, top])."""
    best = torch.topk(z, top, dim=-1)
    return best.indices, torch.softmax(best.values, dim=-1)


def moe_ff(h, w, mlp):
    """w: the layer's 'mlp.*' tensors by short name; mlp: the configuration's entry."""
    T = h.shape[0]
    z = h @ w["router"].T + w["router.b"]
    ids, wt = route_chosen_softmax(z, mlp["router"]["top"])
    out = torch.zeros((T, w["e0.down"].shape[0]), dtype=h.dtype)
    for t in range(T):
        for e, a in zip(ids[t].tolist(), wt[t]):
            out[t] += a * gated_ff(h[t], w["e%d.gate" % e], w["e%d.up" % e], w["e%d.down" % e])
    if mlp.get("shared"):
        out = out + gated_ff(h, w["shared.gate"], w["shared.up"], w["shared.down"])
    return out


def rotate_pairs(x, positions, base, dims):
    """x [T, n, d]: dims 2i and 2i + 1 of the first ``dims`` form a pair, turned by position * base^(-2i / dims)."""
    i = torch.arange(dims // 2, dtype=x.dtype)
    ang = positions.to(x.dtype)[:, None] * torch.pow(torch.tensor(base, dtype=x.dtype), -2.0 * i / dims)[None, :]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def latent_attention(h, w, m, eps):
    """Queries through a normed low-rank vector; keys and values of every head expanded from one normed low-rank vector
    per token, plus one rotated key part that all heads share."""
    T = h.shape[0]
    H, dn, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    cq = rms(h @ w["dq"].T, eps) * w["dq.norm"]
    q = (cq @ w["uq"].T).view(T, H, dn + dr)
    d = h @ w["dkv"].T
    c = rms(d[:, :r], eps) * w["dkv.norm"]
    rot = m["rot"]
    kr = rotate_pairs(d[:, None, r:], pos, rot["base"], rot["dims"])[:, 0]
    qr = rotate_pairs(q[:, :, dn:], pos, rot["base"], rot["dims"])
    k = (c @ w["uk"].T).view(T, H, dn)
    v = (c @ w["uv"].T).view(T, H, dv)
    s = (torch.einsum("ihd,jhd->hij", q[:, :, :dn], k) + torch.einsum("ihd,jd->hij", qr, kr)) * m["scale"]
    s = s.masked_fill(pos[None, :] > pos[:, None], -math.inf)
    o = torch.einsum("hij,jhd->ihd", torch.softmax(s, dim=-1), v)
    o = o * torch.sigmoid(h @ w["g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ w["o"].T


def biased_attention(h, w, m):
    """Grouped queries without rotation: temperature on the queries, capped scores, a penalty on the distance, a softmax
    with a one in the denominator, one gate number per head."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = (h @ w["q"].T + w["q.b"]).view(T, H, d)
    k = (h @ w["k"].T + w["k.b"]).view(T, G, d)
    v = (h @ w["v"].T + w["v.b"]).view(T, G, dv)
    temp = 1.0 + m["q_temp"]["coef"] * torch.log(torch.floor((pos + 1) / m["q_temp"]["every"]).to(h.dtype) + 1.0)
    q = q * temp[:, None, None]
    k = k.repeat_interleave(H // G, dim=1)
    v = v.repeat_interleave(H // G, dim=1)
    s = capped(torch.einsum("ihd,jhd->hij", q, k) * m["scale"], m["softcap"])
    dist = (pos[:, None] - pos[None, :]).clamp(min=0).to(h.dtype)
    s = s - w["r1"][:, None, None] * torch.log1p(w["r2"][:, None, None] * dist[None])
    s = s.masked_fill(pos[None, :] > pos[:, None], -math.inf)
    e = torch.exp(s)                      # (capped scores: no overflow)
    p = e / (1.0 + e.sum(dim=-1, keepdim=True))
    o = torch.einsum("hij,jhd->ihd", p, v)
    o = o * torch.sigmoid(h @ w["g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ w["o"].T


def run_order(n_layers, loop):
    """[(layer, pass number or None)]: the layers of the loop walked ``times`` times, the others once."""
    if not loop:
        return [(i, None) for i in range(n_layers)]
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, None) for i in range(start)]
    for t in range(times):
        order += [(i, t) for i in range(start, stop)]
    return order + [(i, None) for i in range(stop, n_layers)]


# ---- the model ---------------------------------------------------------------------------
class PlainTarunex:
    def __init__(self, config, tensors, dtype=torch.float64):
        self.cfg = config
        self.w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
        self.dtype = dtype

    @classmethod
    def from_folder(cls, folder, dtype=torch.float64):
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json")) as f:
            cfg = json.load(f)
        return cls(cfg, load_file(os.path.join(folder, "model.safetensors")), dtype)

    def sub(self, prefix):
        return {k[len(prefix):]: v for k, v in self.w.items() if k.startswith(prefix)}

    def forward(self, tokens, keep_layers=None):
        """Logits [T, vocab] at every position of one sequence; ``keep_layers``: a list that gets the stream after
        every layer run."""
        cfg, eps = self.cfg, float(self.cfg["norm"]["eps"])
        x0 = self.w["embed"][torch.tensor(tokens, dtype=torch.long)] * float(cfg["embedding"]["scale"])
        x = x0.clone()
        loop = cfg.get("loop")
        for i, t in run_order(len(cfg["layers"]), loop):
            if t is not None and i == loop["start"]:
                if t > 0:
                    x = x + x0
                x = x + self.w["loop.step"][t]
            layer = cfg["layers"][i]
            mw = self.sub("l%d.mix." % i)
            h1 = scalar_norm(x, self.w["l%d.norm1" % i], eps)
            if layer["type"] == "latent_attention":
                y = latent_attention(h1, mw, layer["mixer"], eps)
            elif layer["type"] == "attention":
                y = biased_attention(h1, mw, layer["mixer"])
            else:
                raise ValueError(layer["type"])
            if layer.get("mlp"):
                y = y + moe_ff(scalar_norm(x, self.w["l%d.norm2" % i], eps), self.sub("l%d.mlp." % i), layer["mlp"])
            x = x + y
            if keep_layers is not None:
                keep_layers.append(x.clone())
        z = (scalar_norm(x, self.w["final.norm"], eps) @ self.w["head"].T) * float(cfg["logit_scale"])
        return capped(z, float(cfg["logit_softcap"]))

    def greedy(self, prompt, n):
        toks = list(prompt)
        for _ in range(n):
            toks.append(int(torch.argmax(self.forward(toks)[-1])))
        return toks[len(prompt):]
