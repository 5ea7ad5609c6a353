"""Gated recurrences with a state of fixed size per request.

``MinGRU``: the gates read only the current token, so all of a step's gates come from one product and the
recurrence itself is a scan over the tokens:  z = sigmoid(Wz h + bz), u = Wx h + bx, candidate c = u + 1/2 where
u >= 0 and sigmoid(u) where u < 0;  S_t = (1 - z) S_(t-1) + z c per channel;  output Wo (S_t * silu(Wg h)).  The state
starts at zero, is float32 and lives in the request's slot; everything behind the projections is float32.

``MLSTM`` and ``ChannelDelta`` keep a matrix per head, S [key size, value size], written with k v^T and read with
S^T q.  ``MLSTM``: exponential input gate and sigmoid forget gate in the log domain, both capped by
cap tanh(. / cap), with a running maximum m (from 0) that keeps the exponentials in range:
m = max(f + m', i); S = e^(f + m' - m) S + e^(i - m) k v^T, n likewise with k alone;
o = S^T q / (max(|n . q|, e^-m) + 1e-6), q scaled by 1/sqrt(key size); each head's o over its root mean square, times a
weight, times sigmoid(Wg x), then the output projection.  ``ChannelDelta``: the gated delta rule; q, k and v pass a
short causal convolution per channel and silu, q and k become unit vectors (q also times 1/sqrt(key size));
S = diag(g) S with a decay g = exp(-exp(A_h) softplus(W2 W1 x + bias)) per head and key channel; u = beta (v - S^T k),
beta = sigmoid(Wb x); S += k u^T; o = S^T q; each head's o over its root mean square, times a weight shared by the
heads, times sigmoid(G2 G1 x), then the output projection.  The convolutions' last inputs are state of the request too.
``HeadDelta``: the same rule with ONE decay per head, g = exp(-exp(A_h) softplus(Wa x + bias_h)), and the output gate
silu(Wg x) from a full projection.

``TimeMix``: a state S [key size, key size] per head with a decay per key channel, read BEFORE the token's write except
for the token's own contribution, which enters through a learned bonus u:  o = (S + diag(u) k v^T)^T r;
S = diag(w) S + k v^T.  Every projection reads its own blend of the token's input and the input of the token before it,
x + (x' - x) mu (x' = 0 for a request's first token); w = exp(-exp(W2 tanh(W1 blend_w) + w0)); each head's o over its
root mean square, times a weight, times silu(Wg blend_g), then the output projection.  The input of a request's last
token is state of the request too.
"""
from __future__ import annotations

import numpy as np
import torch

from ..cache.spec import FixedState
from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Mixer

#: tokens of an entry that one thread walks in a row; longer entries are cut, so that a long portion has blocks for
#: the whole device (the pieces' effects on the state are composed, the recurrence being linear in it)
SCAN_PIECE = 32


def scan_pieces_name(piece: int = SCAN_PIECE) -> str:
    return "scan_pieces" if piece == SCAN_PIECE else "scan_pieces_%d" % piece


def plan_scan_pieces(batch, piece: int = SCAN_PIECE) -> None:
    """Adds the step's entries cut into pieces of at most ``piece`` tokens: int32 [4 n] = entry, first row, end row,
    index of the entry's first piece.  Once per step and piece size (``scan_pieces_name``)."""
    name = scan_pieces_name(piece)
    if name in batch.shared:
        return
    lens = batch.lens.astype(np.int64)
    cu = batch.host_array("cu_q").astype(np.int64)
    counts = (lens + piece - 1) // piece
    first = np.zeros(batch.S + 1, dtype=np.int64)
    np.cumsum(counts, out=first[1:])
    n = int(first[-1])
    entry = np.repeat(np.arange(batch.S, dtype=np.int64), counts)
    k = np.arange(n, dtype=np.int64) - first[:-1][entry]
    t0 = cu[:-1][entry] + k * piece
    t1 = np.minimum(t0 + piece, cu[1:][entry])
    batch.add_array(name, np.concatenate([entry, t0, t1, first[:-1][entry]]).astype(np.int32))
    batch.shared[name] = (n, bool((counts > 1).any()))


class MinGRU(Mixer):
    def __init__(self, hidden_size: int, width: int, names=("z", "z.b", "x", "x.b", "g", "o")):
        self.hidden_size, self.width, self.names = hidden_size, width, names
        self.w_zxg = self.w_zxg_tiled = self.w_o = self.w_o_tiled = self.b_z = self.b_x = None

    def weight_specs(self, prefix):
        H, W = self.hidden_size, self.width
        z, zb, x, xb, g, o = (prefix + "." + n for n in self.names)
        return [WeightSpec(z, (W, H)), WeightSpec(zb, (W,), "bias"), WeightSpec(x, (W, H)), WeightSpec(xb, (W,), "bias"),
                WeightSpec(g, (W, H)), WeightSpec(o, (H, W))]

    def bind(self, prefix, weights):
        z, zb, x, xb, g, o = (prefix + "." + n for n in self.names)
        mats = [weights.pop(n) for n in (z, x, g)]
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        # one product for the three projections: rows [z | x | g]
        self.w_zxg, self.w_zxg_tiled = ops.weight_forms(torch.cat(mats, dim=0).contiguous())
        del mats
        self.w_o, self.w_o_tiled = ops.weight_forms(weights.pop(o))
        self.b_z, self.b_x = weights[zb], weights[xb]
        if self.b_z.dtype != self.b_x.dtype:
            self.b_z, self.b_x = self.b_z.float(), self.b_x.float()

    def cache_spec(self):
        return FixedState((self.width,), "float32")

    def plan(self, batch) -> None:
        plan_scan_pieces(batch)

    def plan_arrays(self, entries):
        return {"scan_pieces": 4 * entries}

    def capturable(self, batch):
        return True

    def forward(self, x, batch, cache, store=True):
        if not store:
            raise ValueError("a recurrence cannot run on another layer's state without writing it")
        zxg = ops.linear_few(x, self.w_zxg, self.w_zxg_tiled)
        n, multi = batch.shared["scan_pieces"]
        y = ops.mingru(zxg, self.b_z, self.b_x, cache.state, batch.array("scan_pieces"), n, multi, batch.array("slot_ids"))
        return ops.linear_few(y, self.w_o, self.w_o_tiled)


class MLSTM(Mixer):
    def __init__(self, hidden_size: int, heads: int, dim: int, vdim: int, gate_cap: float, norm_eps: float,
                 names=("q", "k", "v", "g", "o", "norm", "i", "i.b", "f", "f.b")):
        self.hidden_size, self.heads, self.dim, self.vdim = hidden_size, heads, dim, vdim
        self.gate_cap, self.norm_eps, self.names = float(gate_cap), float(norm_eps), names
        if not self.gate_cap > 0.0:
            raise ValueError("the gates' cap must be positive")
        self.w_in = self.w_in_tiled = self.w_gates = self.w_o = self.w_o_tiled = self.b_i = self.b_f = self.norm = None

    def weight_specs(self, prefix):
        W, H, d, dv = self.hidden_size, self.heads, self.dim, self.vdim
        q, k, v, g, o, norm, i, ib, f, fb = (prefix + "." + n for n in self.names)
        return [WeightSpec(q, (H * d, W)), WeightSpec(k, (H * d, W)), WeightSpec(v, (H * dv, W)), WeightSpec(g, (H * dv, W)),
                WeightSpec(o, (W, H * dv)), WeightSpec(norm, (H * dv,), "norm"), WeightSpec(i, (H, W)), WeightSpec(ib, (H,), "bias"),
                WeightSpec(f, (H, W)), WeightSpec(fb, (H,), "bias")]

    def bind(self, prefix, weights):
        q, k, v, g, o, norm, i, ib, f, fb = (prefix + "." + n for n in self.names)
        mats = [weights.pop(n) for n in (q, k, v, g)]
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        # one product for the four wide projections: rows [q | k | v | g]; the two gates' products, which enter the
        # recurrence's exponentials, come from a second, small product whose result stays float32
        self.w_in, self.w_in_tiled = ops.weight_forms(torch.cat(mats, dim=0).contiguous())
        del mats
        gi, gf = weights.pop(i), weights.pop(f)
        if gi.dtype != gf.dtype:
            gi, gf = gi.float(), gf.float()
        self.w_gates = torch.cat([gi, gf], dim=0).contiguous()
        self.w_o, self.w_o_tiled = ops.weight_forms(weights.pop(o))
        small = [weights[ib], weights[fb], weights[norm]]
        if len({t.dtype for t in small}) > 1:
            small = [t.float() for t in small]
        self.b_i, self.b_f, self.norm = small

    def cache_spec(self):
        return FixedState((ops.mlstm_state_size(self.heads, self.dim, self.vdim),), "float32")

    #: tokens of an entry that one wave walks in a row; longer entries are cut (their pieces' effects on the state are
    #: composed: with the running maximum known, the state is linear in itself)
    PIECE = 64

    def plan(self, batch) -> None:
        plan_scan_pieces(batch, self.PIECE)

    def plan_arrays(self, entries):
        return {scan_pieces_name(self.PIECE): 4 * entries}

    def capturable(self, batch):
        return True

    def forward(self, x, batch, cache, store=True):
        if not store:
            raise ValueError("a recurrence cannot run on another layer's state without writing it")
        H, d, dv = self.heads, self.dim, self.vdim
        proj = ops.linear_few(x, self.w_in, self.w_in_tiled)
        gates = ops.linear(x, self.w_gates, torch.float32)
        name = scan_pieces_name(self.PIECE)
        n, multi = batch.shared[name]
        y = ops.mlstm(proj, 0, H * d, 2 * H * d, 2 * H * d + H * dv, gates, self.b_i, self.b_f, self.gate_cap, self.norm, self.norm_eps,
                      cache.state, batch.array("cu_q"), batch.array("slot_ids"), H, d, dv, pieces=(batch.array(name), n, multi))
        return ops.linear_few(y, self.w_o, self.w_o_tiled)


class ChannelDelta(Mixer):
    def __init__(self, hidden_size: int, heads: int, kv_heads: int, dim: int, vdim: int, conv: int, norm_eps: float,
                 decay_rank: int = None, gate_rank: int = None,
                 names=("q", "k", "v", "b", "a1", "g1", "a2", "g2", "o", "q.conv", "k.conv", "v.conv", "A_log", "dt_bias", "norm")):
        """``decay_rank``, ``gate_rank``: inner sizes of the two low-rank projections; None: whatever the stored
        tensors have (a model folder is then needed: random weights cannot be drawn for an unknown size)."""
        if heads % kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        self.hidden_size, self.heads, self.kv_heads, self.dim, self.vdim, self.conv = hidden_size, heads, kv_heads, dim, vdim, conv
        self.norm_eps, self.names = float(norm_eps), names
        self.rank_a, self.rank_g = (-1 if decay_rank is None else decay_rank), (-1 if gate_rank is None else gate_rank)
        if not 1 <= conv <= 8:
            raise ValueError("the short convolution has 1 to 8 taps")
        self.w_in = self.w_in_tiled = self.w_small = self.w_a2 = self.w_g2 = self.w_g2_tiled = self.w_o = self.w_o_tiled = None
        self.taps = self.a_log = self.dt_bias = self.norm = None

    def _channels(self):
        return 2 * self.kv_heads * self.dim + self.heads * self.vdim

    def weight_specs(self, prefix):
        W, H, G, d, dv, n = self.hidden_size, self.heads, self.kv_heads, self.dim, self.vdim, self.conv
        q, k, v, b, a1, g1, a2, g2, o, qc, kc, vc, alog, dtb, norm = (prefix + "." + x for x in self.names)
        ra, rg = self.rank_a, self.rank_g
        return [WeightSpec(q, (G * d, W)), WeightSpec(k, (G * d, W)), WeightSpec(v, (H * dv, W)), WeightSpec(b, (H, W)),
                WeightSpec(a1, (ra, W)), WeightSpec(g1, (rg, W)), WeightSpec(a2, (H * d, ra)), WeightSpec(g2, (H * dv, rg)),
                WeightSpec(o, (W, H * dv)), WeightSpec(qc, (G * d, n), "bias"), WeightSpec(kc, (G * d, n), "bias"),
                WeightSpec(vc, (H * dv, n), "bias"), WeightSpec(alog, (H,), "bias"), WeightSpec(dtb, (H * d,), "bias"),
                WeightSpec(norm, (dv,), "norm")]

    def bind(self, prefix, weights):
        q, k, v, b, a1, g1, a2, g2, o, qc, kc, vc, alog, dtb, norm = (prefix + "." + x for x in self.names)
        mats = [weights.pop(n) for n in (q, k, v, g1)]
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        if weights[a2].shape[1] != weights[a1].shape[0] or weights[g2].shape[1] != mats[3].shape[0]:
            raise ValueError("%s: the inner sizes of the low-rank projections do not fit each other" % prefix)
        # one product for the wide projections and the output gate's inner one: rows [q | k | v | g1]; what enters the
        # recurrence's exponentials (beta, the decay's inner projection) comes from a second product that stays float32
        self.w_in, self.w_in_tiled = ops.weight_forms(torch.cat(mats, dim=0).contiguous())
        del mats
        small = [weights.pop(b), weights.pop(a1)]
        if small[0].dtype != small[1].dtype:
            small = [t.float() for t in small]
        self.w_small = torch.cat(small, dim=0).contiguous()
        self.w_a2 = weights.pop(a2)
        self.w_g2, self.w_g2_tiled = ops.weight_forms(weights.pop(g2))
        self.w_o, self.w_o_tiled = ops.weight_forms(weights.pop(o))
        taps = [weights[n] for n in (qc, kc, vc)]
        vecs = [weights[alog], weights[dtb], weights[norm]]
        if len({t.dtype for t in taps + vecs}) > 1:
            taps, vecs = [t.float() for t in taps], [t.float() for t in vecs]
        self.taps = torch.cat(taps, dim=0).contiguous()
        self.a_log, self.dt_bias, self.norm = vecs

    def cache_spec(self):
        H, d, dv = self.heads, self.dim, self.vdim
        return FixedState((H * d * dv + (self.conv - 1) * self._channels(),), "float32")

    def capturable(self, batch):
        return True

    def forward(self, x, batch, cache, store=True):
        if not store:
            raise ValueError("a recurrence cannot run on another layer's state without writing it")
        H, G, d, dv, C = self.heads, self.kv_heads, self.dim, self.vdim, self._channels()
        proj = ops.linear_few(x, self.w_in, self.w_in_tiled)
        small = ops.linear(x, self.w_small, torch.float32)                    # [beta | a1], float32 sums kept
        beta_pre = small[:, :H].contiguous()
        # (the inner projection's result is an activation: it takes the activation dtype on its way into the outer one)
        dec_pre = ops.linear(small[:, H:].to(self.w_a2.dtype).contiguous(), self.w_a2, torch.float32)
        gate = ops.linear_few(proj[:, C:].contiguous(), self.w_g2, self.w_g2_tiled)
        cu_q, slots = batch.array("cu_q"), batch.array("slot_ids")
        qkv = ops.causal_conv_silu(proj[:, :C], self.taps, cache.state, H * d * dv, batch.array("token_entry"), cu_q, slots)
        y = ops.delta_rule(qkv, beta_pre, dec_pre, self.a_log, self.dt_bias, gate, self.norm, self.norm_eps, cache.state, cu_q, slots,
                           H, G, d, dv)
        return ops.linear_few(y, self.w_o, self.w_o_tiled)


class HeadDelta(Mixer):
    """The gated delta rule with one decay per head and a full output gate (see the module's text)."""

    def __init__(self, hidden_size: int, heads: int, kv_heads: int, dim: int, vdim: int, conv: int, norm_eps: float,
                 names=("q", "k", "v", "b", "a", "g", "o", "q.conv", "k.conv", "v.conv", "A_log", "dt_bias", "norm")):
        if heads % kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        if not 1 <= conv <= 8:
            raise ValueError("the short convolution has 1 to 8 taps")
        self.hidden_size, self.heads, self.kv_heads, self.dim, self.vdim, self.conv = hidden_size, heads, kv_heads, dim, vdim, conv
        self.norm_eps, self.names = float(norm_eps), names
        self.w_in = self.w_in_tiled = self.w_small = self.w_o = self.w_o_tiled = None
        self.taps = self.a_log = self.dt_bias = self.norm = None

    def _channels(self):
        return 2 * self.kv_heads * self.dim + self.heads * self.vdim

    def weight_specs(self, prefix):
        W, H, G, d, dv, n = self.hidden_size, self.heads, self.kv_heads, self.dim, self.vdim, self.conv
        q, k, v, b, a, g, o, qc, kc, vc, alog, dtb, norm = (prefix + "." + x for x in self.names)
        return [WeightSpec(q, (G * d, W)), WeightSpec(k, (G * d, W)), WeightSpec(v, (H * dv, W)), WeightSpec(b, (H, W)),
                WeightSpec(a, (H, W)), WeightSpec(g, (H * dv, W)), WeightSpec(o, (W, H * dv)), WeightSpec(qc, (G * d, n), "bias"),
                WeightSpec(kc, (G * d, n), "bias"), WeightSpec(vc, (H * dv, n), "bias"), WeightSpec(alog, (H,), "bias"),
                WeightSpec(dtb, (H,), "bias"), WeightSpec(norm, (dv,), "norm")]

    def bind(self, prefix, weights):
        q, k, v, b, a, g, o, qc, kc, vc, alog, dtb, norm = (prefix + "." + x for x in self.names)
        mats = [weights.pop(n) for n in (q, k, v, g)]
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        # one product for the wide projections: rows [q | k | v | gate]; what enters the recurrence's exponentials (beta,
        # the decay) comes from a second, small product that stays float32
        self.w_in, self.w_in_tiled = ops.weight_forms(torch.cat(mats, dim=0).contiguous())
        del mats
        small = [weights.pop(b), weights.pop(a)]
        if small[0].dtype != small[1].dtype:
            small = [t.float() for t in small]
        self.w_small = torch.cat(small, dim=0).contiguous()
        self.w_o, self.w_o_tiled = ops.weight_forms(weights.pop(o))
        taps = [weights[n] for n in (qc, kc, vc)]
        vecs = [weights[alog], weights[dtb], weights[norm]]
        if len({t.dtype for t in taps + vecs}) > 1:
            taps, vecs = [t.float() for t in taps], [t.float() for t in vecs]
        self.taps = torch.cat(taps, dim=0).contiguous()
        self.a_log, self.dt_bias, self.norm = vecs

    def cache_spec(self):
        H, d, dv = self.heads, self.dim, self.vdim
        return FixedState((H * d * dv + (self.conv - 1) * self._channels(),), "float32")

    def capturable(self, batch):
        return True

    def forward(self, x, batch, cache, store=True):
        if not store:
            raise ValueError("a recurrence cannot run on another layer's state without writing it")
        H, G, d, dv, C = self.heads, self.kv_heads, self.dim, self.vdim, self._channels()
        proj = ops.linear_few(x, self.w_in, self.w_in_tiled)
        small = ops.linear(x, self.w_small, torch.float32)                    # [beta | decay], float32 sums kept
        beta_pre, dec_pre = small[:, :H], small[:, H:]                        # (the walk's kernels read them where they lie)
        cu_q, slots = batch.array("cu_q"), batch.array("slot_ids")
        qkv = ops.causal_conv_silu(proj[:, :C], self.taps, cache.state, H * d * dv, batch.array("token_entry"), cu_q, slots)
        y = ops.delta_rule(qkv, beta_pre, dec_pre, self.a_log, self.dt_bias, proj[:, C:], self.norm, self.norm_eps, cache.state, cu_q, slots,
                           H, G, d, dv, gate_act="silu")
        return ops.linear_few(y, self.w_o, self.w_o_tiled)


class TimeMix(Mixer):
    """Token shift and a per-head state with a decay per key channel and a bonus for the current token (see the module's
    text).  Tensors: ``mu.r/k/v/g/w [W]``, ``r``, ``k``, ``v``, ``g [H d, W]``, ``w1 [rank, W]``, ``w2 [H d, rank]``,
    ``w0 [H d]``, ``u [H, d]``, ``norm [H d]``, ``o [W, H d]``; the decay's inner size is the stored tensors'."""

    BLENDS = ("r", "k", "v", "g", "w")

    def __init__(self, hidden_size: int, heads: int, dim: int, norm_eps: float, decay_rank: int = None,
                 names=("mu.%s", "r", "k", "v", "g", "w1", "w2", "w0", "u", "norm", "o")):
        self.hidden_size, self.heads, self.dim, self.norm_eps, self.names = hidden_size, heads, dim, float(norm_eps), names
        self.rank = -1 if decay_rank is None else decay_rank
        self.mu = self.w_r = self.w_k = self.w_v = self.w_g = self.w_1 = self.w_2 = self.w_o = None
        self.w0 = self.u = self.norm = None

    def weight_specs(self, prefix):
        W, N = self.hidden_size, self.heads * self.dim
        mu, r, k, v, g, w1, w2, w0, u, norm, o = (prefix + "." + x for x in self.names)
        specs = [WeightSpec(mu % b, (W,), "bias") for b in self.BLENDS]
        specs += [WeightSpec(n, (N, W)) for n in (r, k, v, g)]
        specs += [WeightSpec(w1, (self.rank, W)), WeightSpec(w2, (N, self.rank)), WeightSpec(w0, (N,), "bias"),
                  WeightSpec(u, (self.heads, self.dim), "bias"), WeightSpec(norm, (N,), "norm"), WeightSpec(o, (W, N))]
        return specs

    def bind(self, prefix, weights):
        mu, r, k, v, g, w1, w2, w0, u, norm, o = (prefix + "." + x for x in self.names)
        if weights[w2].shape[1] != weights[w1].shape[0]:
            raise ValueError("%s: the inner sizes of the decay's two projections do not fit each other" % prefix)
        mus = [weights[mu % b] for b in self.BLENDS]
        vecs = [weights[w0], weights[u].reshape(-1), weights[norm]]
        if len({t.dtype for t in mus + vecs}) > 1:
            mus, vecs = [t.float() for t in mus], [t.float() for t in vecs]
        self.mu = torch.stack(mus).contiguous()
        self.w0, self.u, self.norm = (t.contiguous() for t in vecs)
        self.w_r, self.w_k, self.w_v, self.w_g = (ops.weight_forms(weights.pop(n)) for n in (r, k, v, g))
        # the decay's two products keep their float32 sums: what they give enters two exponentials
        self.w_1, self.w_2 = weights.pop(w1), weights.pop(w2)
        self.w_o = ops.weight_forms(weights.pop(o))

    def cache_spec(self):
        return FixedState((self.heads * self.dim * self.dim + self.hidden_size,), "float32")

    def capturable(self, batch):
        return True

    def forward(self, x, batch, cache, store=True):
        if not store:
            raise ValueError("a recurrence cannot run on another layer's state without writing it")
        H, d = self.heads, self.dim
        cu_q, slots = batch.array("cu_q"), batch.array("slot_ids")
        blends = ops.token_shift(x, self.mu, cache.state, H * d * d, batch.array("token_entry"), cu_q, slots)      # [5, T, W]
        r, k, v, g = (ops.linear_few(blends[i], w[0], w[1]) for i, w in enumerate((self.w_r, self.w_k, self.w_v, self.w_g)))
        # (the inner projection's result is an activation: it takes the outer matrix's dtype on its way into that product)
        inner = ops.tanh_cast(ops.linear(blends[4], self.w_1, torch.float32), self.w_2.dtype)
        dec_pre = ops.linear(inner, self.w_2, torch.float32)
        y = ops.time_mix(r, k, v, dec_pre, self.w0, self.u, g, self.norm, self.norm_eps, cache.state, cu_q, slots, H, d)
        return ops.linear_few(y, self.w_o[0], self.w_o[1])
