"""Plain, slow Meronex forward pass: whole sequences, no cache, one function per mechanism.

Meronex is a pre-norm decoder: x += m * gate1 * mixer(norm1(x)), x += m * gate2 * ff(norm2(x)), with a constant m,
norms that work on consecutive groups of the vector, and a sigmoid gate (a full matrix and a bias on the normed
input) on every sublayer's result.  A layer's token mixer is one of three: a matrix memory with exponential input gate
and a running maximum (mLSTM); a gated delta rule with short causal convolutions and one decay per head; or two
mixers side by side on the same input, a grouped-query attention (rotation with rescaled frequencies, values normed
per head, scores capped by a tanh) and a time mix with token shift and a decay per key channel, whose results are
normed over the width each and averaged.  The feed-forward is a mixture of experts with sigmoid scores that multiply
the chosen experts' INPUT, and a clamped, shifted activation.

This file shares no code with the ``spyinfer_amd`` package.  It takes a configuration as a dictionary and the tensors
as a dictionary of CPU tensors, and computes in ``dtype`` (float64 by default).
"""
import json
import math
import os

import torch


# ---- pieces ------------------------------------------------------------------------------
def rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def grouped_norm(x, w, eps, groups):
    """The vector in ``groups`` equal consecutive parts, each over its own root mean square; then the weight."""
    T, W = x.shape
    return rms(x.view(T, groups, W // groups), eps).reshape(T, W) * w


def silu(z):
    return z * torch.sigmoid(z)


def result_gate(h, w, b):
    """What multiplies a sublayer's result: sigmoid(W h + b), h the sublayer's input."""
    return torch.sigmoid(h @ w.T + b)


def clamped_expert(h, gate, up, down, limit):
    g = torch.clamp(h @ gate.T, max=limit)
    u = torch.clamp(h @ up.T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def sigmoid_route(z, top):
    """Router logits z [T, E] -> (chosen experts [T, top], their weights [T, top]): the largest sigmoid scores, as they are."""
    s = torch.sigmoid(z)
    ids = torch.topk(s, top, dim=-1).indices
    return ids, torch.gather(s, 1, ids)


def moe_ff(h, w, cfg):
    """w: the layer's 'mlp.*' tensors by short name.  The weight multiplies the expert's input."""
    ids, wt = sigmoid_route(h @ w["router"].T, cfg["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(ids.shape[1]):
            e = int(ids[t, j])
            out[t] += clamped_expert(wt[t, j] * h[t:t + 1], w["e%d.gate" % e], w["e%d.up" % e], w["e%d.down" % e], cfg["expert"]["limit"])[0]
    return out


def ramped_frequencies(rot, dtype=torch.float64):
    """(frequencies of the pairs, factor on cos and sin).  f_i = base^(-2i/dims); with a scaling, frequencies are
    divided by the factor along a linear ramp over the pair index between the pairs that make ``fast`` and ``slow`` turns
    in ``original`` positions."""
    dims, base = rot["dims"], float(rot["base"])
    i = torch.arange(dims // 2, dtype=dtype)
    f = torch.tensor(base, dtype=dtype) ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def index_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(index_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(index_of(float(sc["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_half(x, positions, freq, mag, dims):
    """x [T, heads, d]: dimension i pairs with i + dims/2 within the first ``dims``; the rest passes."""
    half = dims // 2
    ang = positions.to(freq.dtype)[:, None] * freq[None, :]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


def capped_attention(h, w, cfg, eps):
    """Grouped-query attention over all earlier tokens: rotated q and k, values over their root mean square per head,
    scores times ``scale`` and then capped by cap tanh(. / cap), softmax, output projection."""
    T = h.shape[0]
    H, G, d, dv = cfg["heads"], cfg.get("kv_heads") or cfg["heads"], cfg["dim"], cfg["vdim"]
    q = (h @ w["q"].T).view(T, H, d)
    k = (h @ w["k"].T).view(T, G, d)
    v = rms((h @ w["v"].T).view(T, G, dv), eps)
    rot = cfg.get("rot")
    if rot:
        freq, mag = ramped_frequencies(rot, h.dtype)
        pos = torch.arange(T)
        q, k = rotate_half(q, pos, freq, mag, rot["dims"]), rotate_half(k, pos, freq, mag, rot["dims"])
    out = torch.zeros((T, H, dv), dtype=h.dtype)
    cap = cfg.get("softcap")
    for t in range(T):
        for hd in range(H):
            g = hd // (H // G)
            sc = (k[:t + 1, g] @ q[t, hd]) * cfg["scale"]
            if cap:
                sc = cap * torch.tanh(sc / cap)
            out[t, hd] = torch.softmax(sc, dim=0) @ v[:t + 1, g]
    return out.reshape(T, H * dv) @ w["o"].T


def time_mix(h, w, cfg, eps):
    """Token shift, then per head a state S [d, d]: o_t = (S + diag(u) k v^T)^T r; S = diag(w_t) S + k v^T."""
    T, W = h.shape
    H, d = cfg["heads"], cfg["dim"]
    prev = torch.cat([torch.zeros((1, W), dtype=h.dtype), h[:-1]], dim=0)

    def mixed(name):
        return h + (prev - h) * w["mu." + name]
    r = (mixed("r") @ w["r"].T).view(T, H, d)
    k = (mixed("k") @ w["k"].T).view(T, H, d)
    v = (mixed("v") @ w["v"].T).view(T, H, d)
    gate = silu(mixed("g") @ w["g"].T)
    decay = torch.exp(-torch.exp(torch.tanh(mixed("w") @ w["w1"].T) @ w["w2"].T + w["w0"])).view(T, H, d)
    u = w["u"].view(H, d)
    S = torch.zeros((H, d, d), dtype=h.dtype)
    out = torch.zeros((T, H, d), dtype=h.dtype)
    for t in range(T):
        kv = k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hi,hij->hj", r[t], S + u[:, :, None] * kv)
        S = decay[t][:, :, None] * S + kv
    y = rms(out, eps).reshape(T, H * d) * w["norm"] * gate
    return y @ w["o"].T


def side_by_side(h, w, cfg, eps):
    """Two mixers on one input; each result normed over the width with a plain weight; half their sum."""
    left = {k[5:]: v for k, v in w.items() if k.startswith("left.")}
    right = {k[6:]: v for k, v in w.items() if k.startswith("right.")}
    a = rms(capped_attention(h, left, cfg["left"], eps), eps) * left["out"]
    b = rms(time_mix(h, right, cfg["right"], eps), eps) * right["out"]
    return 0.5 * (a + b)


def mlstm(h, w, cfg, eps):
    """Matrix memory with exponential gates in the log domain and a running maximum that starts at 0."""
    T = h.shape[0]
    H, d, dv, cap = cfg["heads"], cfg["dim"], cfg["vdim"], float(cfg["gate_cap"])
    q = (h @ w["q"].T).view(T, H, d) * d ** -0.5
    k = (h @ w["k"].T).view(T, H, d)
    v = (h @ w["v"].T).view(T, H, dv)
    ig = cap * torch.tanh((h @ w["i"].T + w["i.b"]) / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ w["f"].T + w["f.b"]) / cap))
    S = torch.zeros((H, d, dv), dtype=h.dtype)
    n = torch.zeros((H, d), dtype=h.dtype)
    m = torch.zeros((H,), dtype=h.dtype)
    out = torch.zeros((T, H, dv), dtype=h.dtype)
    for t in range(T):
        m_new = torch.maximum(fg[t] + m, ig[t])
        a, b = torch.exp(fg[t] + m - m_new), torch.exp(ig[t] - m_new)
        S = a[:, None, None] * S + b[:, None, None] * (k[t][:, :, None] * v[t][:, None, :])
        n = a[:, None] * n + b[:, None] * k[t]
        m = m_new
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        out[t] = torch.einsum("hi,hij->hj", q[t], S) / den[:, None]
    y = rms(out, eps).reshape(T, H * dv) * w["norm"] * torch.sigmoid(h @ w["g"].T)
    return y @ w["o"].T


def causal_conv(x, taps):
    """x [T, C], taps [C, n]: y[t] = sum_j taps[:, j] x[t - (n - 1) + j], zeros before the start."""
    T, C = x.shape
    n = taps.shape[1]
    padded = torch.cat([torch.zeros((n - 1, C), dtype=x.dtype), x], dim=0)
    y = torch.zeros_like(x)
    for j in range(n):
        y += padded[j:j + T] * taps[:, j]
    return y


def gated_delta(h, w, cfg, eps):
    """Gated delta rule, one decay per head: S = g S; u = beta (v - S^T k); S += k u^T; o = S^T q."""
    T = h.shape[0]
    H, G, d, dv = cfg["heads"], cfg.get("kv_heads") or cfg["heads"], cfg["dim"], cfg["vdim"]
    q = silu(causal_conv(h @ w["q"].T, w["q.conv"])).view(T, G, d)
    k = silu(causal_conv(h @ w["k"].T, w["k.conv"])).view(T, G, d)
    v = silu(causal_conv(h @ w["v"].T, w["v.conv"])).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w["b"].T)
    g = torch.exp(-torch.exp(w["A_log"]) * torch.nn.functional.softplus(h @ w["a"].T + w["dt_bias"]))
    S = torch.zeros((H, d, dv), dtype=h.dtype)
    out = torch.zeros((T, H, dv), dtype=h.dtype)
    for t in range(T):
        for hd in range(H):
            kv = hd // (H // G)
            S[hd] = g[t, hd] * S[hd]
            u = beta[t, hd] * (v[t, hd] - S[hd].T @ k[t, kv])
            S[hd] = S[hd] + torch.outer(k[t, kv], u)
            out[t, hd] = S[hd].T @ q[t, kv]
    y = (rms(out, eps) * w["norm"]).reshape(T, H * dv) * silu(h @ w["g"].T)
    return y @ w["o"].T


MIXERS = {"mlstm": mlstm, "delta": gated_delta, "parallel": side_by_side}


# ---- the model -----------------------------------------------------------------------------
class PlainMeronex:
    def __init__(self, config, tensors, dtype=torch.float64):
        self.cfg = config
        self.dtype = dtype
        self.w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}

    @classmethod
    def from_folder(cls, folder, dtype=torch.float64):
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json")) as f:
            config = json.load(f)
        return cls(config, load_file(os.path.join(folder, "model.safetensors")), dtype)

    def _sub(self, prefix):
        return {k[len(prefix):]: v for k, v in self.w.items() if k.startswith(prefix)}

    def forward(self, tokens, layers_out=None):
        """Logits [T, vocab] of a whole sequence; ``layers_out``: a list that receives the stream after every layer."""
        cfg, w = self.cfg, self.w
        eps, groups, m = float(cfg["norm"]["eps"]), int(cfg["norm"]["groups"]), float(cfg["residual_mult"])
        x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
        for i, layer in enumerate(cfg["layers"]):
            p = "l%d." % i
            h = grouped_norm(x, w[p + "norm1"], eps, groups)
            y = MIXERS[layer["type"]](h, self._sub(p + "mix."), layer["mixer"], eps)
            x = x + m * y * result_gate(h, w[p + "rg1"], w[p + "rg1.b"])
            if layer.get("mlp"):
                h = grouped_norm(x, w[p + "norm2"], eps, groups)
                y = moe_ff(h, self._sub(p + "mlp."), layer["mlp"])
                x = x + m * y * result_gate(h, w[p + "rg2"], w[p + "rg2.b"])
            if layers_out is not None:
                layers_out.append(x.clone())
        return grouped_norm(x, w["final.norm"], eps, groups) @ w["head"].T

    def greedy(self, prompt, n):
        toks = list(prompt)
        out = []
        for _ in range(n):
            nxt = int(torch.argmax(self.forward(toks)[-1]))
            out.append(nxt)
            toks.append(nxt)
        return out
