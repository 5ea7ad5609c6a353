"""Latent attention: keys and values of all heads are expanded from one low-rank vector per token.

Per token the layer projects  q = Wq h  (per head ``dim`` unrotated and ``rot_dim`` rotated values) and
d = Wdkv h  (``kv_rank + rot_dim`` values): c = rmsnorm(d[:kv_rank]) * w is the latent, d[kv_rank:] rotated is a key
part that all heads share.  Head h has keys Wuk_h c and values Wuv_h c; its score against token j is
(q_h[:dim] . Wuk_h c_j + rot(q_h[dim:]) . kr_j) * scale.  Only c and kr are cached, one row per token
(``PagedRows``), and keys and values are never formed: the query is taken through Wuk_h once
(qa_h = Wuk_h^T q_h[:dim], so that the score is qa_h . c_j + ...), the attention sums latents, and Wuv_h is applied to the
sum.  Options: a sliding window (position i sees j with 0 <= i - j < window), a learned sink per head that adds
exp(sink_h) to the softmax's denominator, and ``shares_cache``: the layer has no Wdkv and reads the rows of another
layer (run order: ``LayerCall(layer, cache=that layer's, store=False)``).  ``q_rank``: the queries too pass through a
low-rank vector, q = Wuq (rmsnorm(Wdq h) * w).  ``gate``: every head's result is multiplied by one number,
sigmoid(Wg h)_h.  A rotary encoding with interleaved pairs is taken as it says.
"""
from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from ..cache.spec import PagedRows
from ..kernels import ops
from ..weights.loader import WeightSpec
from .attention import attention_meta
from .base import Mixer
from .rotary import RotaryEmbedding


class LatentAttention(Mixer):
    def __init__(self, hidden_size: int, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int, scale: float, norm_eps: float,
                 position: Optional[RotaryEmbedding] = None, window: Optional[int] = None, cache_window: Optional[int] = -1,
                 sink: bool = True, shares_cache: bool = False,
                 names=("q", "dkv", "dkv.norm", "uk", "uv", "sink", "o"), q_rank: Optional[int] = None, gate: bool = False,
                 more_names=("dq", "dq.norm", "uq", "g")):
        """``window``: what this layer's queries see; ``cache_window``: what the cache rows are kept for, the largest
        window of the layers that read them (None = everything; -1 = this layer's own window).  ``position``: a rotary
        encoding over the rotated part (its ``rotary_dim`` <= rot_dim values are rotated).  ``q_rank``: size of the
        queries' low-rank vector (tensors ``dq``, ``dq.norm``, ``uq`` in place of ``q``; the norm has the layer's eps).
        ``gate``: a matrix ``g [heads, hidden]``, one sigmoid number per head on the head's result."""
        self.q_rank, self.has_gate, self.more_names = q_rank, bool(gate), more_names
        self.w_uq = self.w_uq_tiled = self.q_norm = None
        self.hidden_size, self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank = hidden_size, heads, dim, rot_dim, vdim, kv_rank
        self.scale, self.norm_eps = float(scale), float(norm_eps)
        self.position, self.window = position, window
        self.cache_window = window if cache_window == -1 else cache_window
        if self.cache_window is not None and (window is None or window > self.cache_window):
            raise ValueError("the cache rows are kept for %r tokens, the layer's window is %r" % (self.cache_window, window))
        self.has_sink, self.shares_cache, self.names = sink, shares_cache, names
        self.w_in = self.w_in_tiled = self.w_uk = self.w_uv = self.w_o = self.w_o_tiled = self.c_norm = self.sink = None

    # ---- weights ---------------------------------------------------------
    def _names(self, prefix):
        return tuple(prefix + "." + n for n in self.names)

    def weight_specs(self, prefix):
        q, dkv, dkv_norm, uk, uv, sink, o = self._names(prefix)
        H, nh, dn, dr, dv, r = self.hidden_size, self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank
        dq, dq_norm, uq, g = (prefix + "." + n for n in self.more_names)
        if self.q_rank:
            specs = [WeightSpec(dq, (self.q_rank, H)), WeightSpec(dq_norm, (self.q_rank,), "norm"), WeightSpec(uq, (nh * (dn + dr), self.q_rank))]
        else:
            specs = [WeightSpec(q, (nh * (dn + dr), H))]
        if self.has_gate:
            specs.append(WeightSpec(g, (nh, H)))
        if not self.shares_cache:
            specs += [WeightSpec(dkv, (r + dr, H)), WeightSpec(dkv_norm, (r,), "norm")]
        specs += [WeightSpec(uk, (nh * dn, r)), WeightSpec(uv, (nh * dv, r))]
        if self.has_sink:
            specs.append(WeightSpec(sink, (nh,), "bias"))
        specs.append(WeightSpec(o, (H, nh * dv)))
        return specs

    def bind(self, prefix, weights):
        q, dkv, dkv_norm, uk, uv, sink, o = self._names(prefix)
        dq, dq_norm, uq, g = (prefix + "." + n for n in self.more_names)
        if self.q_rank:
            w_q = weights.pop(dq)
            self.q_norm = weights[dq_norm]
            self.w_uq, self.w_uq_tiled = ops.weight_forms(weights.pop(uq))
        else:
            w_q = weights.pop(q)
        # one product of the mixer's input: rows [q of all heads (or their low-rank vector) | dkv | gate], filled up with
        # zero rows to whole tiles of 16
        mats = [w_q]
        if not self.shares_cache:
            mats.append(weights.pop(dkv))
            self.c_norm = weights[dkv_norm]
        if self.has_gate:
            mats.append(weights.pop(g))
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        rows = sum(m.shape[0] for m in mats)
        if len(mats) > 1 and rows % 16:
            mats.append(torch.zeros((-rows % 16, mats[0].shape[1]), dtype=mats[0].dtype, device=mats[0].device))
        w_in = torch.cat(mats, dim=0).contiguous() if len(mats) > 1 else w_q
        del mats
        self.w_in, self.w_in_tiled = ops.weight_forms(w_in)
        nh, dn, dv, r = self.heads, self.dim, self.vdim, self.kv_rank
        # both expansion matrices per head with the summed index innermost: [H, kv_rank, dim] (transposed once, here) for
        # the queries' way through the keys' expansion, [H, vdim, kv_rank] (as stored) for the summed latents' way out
        self.w_uk = weights.pop(uk).view(nh, dn, r).transpose(1, 2).contiguous()
        self.w_uv = weights.pop(uv).view(nh, dv, r).contiguous()
        self.w_o, self.w_o_tiled = ops.weight_forms(weights.pop(o))
        if self.has_sink:
            self.sink = weights[sink]
        if self.position is not None:
            self.position.prepare(self.w_uk.device, 0)

    # ---- cache -----------------------------------------------------------
    def cache_spec(self):
        return PagedRows(self.kv_rank + self.rot_dim, self.cache_window)

    def capturable(self, batch):
        return True

    def plan(self, batch) -> None:
        """The step's query rows, (token, head) pairs of each entry, cut into tiles for the MFMA kernel, and the number
        of parts of a tile's keys (a launch shape: it goes into a captured step's key)."""
        if not ops.latent_attention_mfma_ok(batch.act_dtype, self.kv_rank, self.kv_rank + self.rot_dim):
            return
        note = ("latent_tiles", self.heads)
        if note not in batch.shared:
            rows = batch.lens.astype(np.int64) * self.heads
            size = ops.latent_tile_rows(int(rows.sum()))
            counts = (rows + size - 1) // size
            entry = np.repeat(np.arange(batch.S, dtype=np.int64), counts)
            first = np.zeros(batch.S + 1, dtype=np.int64)
            np.cumsum(counts, out=first[1:])
            row0 = (np.arange(int(first[-1]), dtype=np.int64) - first[:-1][entry]) * size
            batch.add_array("latent_tile_entry_%d" % self.heads, entry)
            batch.add_array("latent_tile_row0_%d" % self.heads, row0)
            batch.shared[note] = int(first[-1])
            batch.shared[("latent_tile_rows", self.heads)] = size
        keys = batch.max_kv_len if self.window is None else min(batch.max_kv_len, self.window + batch.max_q_len - 1)
        parts = ops.latent_key_parts(batch.shared[note], keys)
        batch.shared[("latent_parts", self.heads, self.window)] = parts
        batch.add_graph_key("latent_parts_%d_%s" % (self.heads, self.window), parts)

    def plan_arrays(self, entries):
        n = entries * -(-self.heads // ops.LATENT_TILE_ROWS)
        return {"latent_tile_entry_%d" % self.heads: n, "latent_tile_row0_%d" % self.heads: n}

    def _frequencies(self):
        if self.position is None:
            return None, 1.0, 0
        return self.position.frequencies()

    # ---- step ------------------------------------------------------------
    def forward(self, x, batch, cache, store=True):
        if store == self.shares_cache:
            raise ValueError("a latent attention layer %s" % ("without a projection of its own cannot fill a cache" if store
                                                             else "with a projection of its own was told to read another's cache"))
        nh, dn, dr, dv, r = self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank
        T = x.shape[0]
        qd = ops.linear_few(x, self.w_in, self.w_in_tiled)
        # where the parts of the product's rows begin: the queries (or their low-rank vector), the latent's rows, the gate
        nq = self.q_rank if self.q_rank else nh * (dn + dr)
        g0 = nq + (0 if self.shares_cache else r + dr)
        if self.q_rank:
            # the queries from their normed low-rank vector (the norm reads its rows inside the wider product)
            q_rows = ops.linear_few(ops.rms_norm(qd[:, :nq], self.q_norm, self.norm_eps), self.w_uq, self.w_uq_tiled)
        else:
            q_rows = qd
        freq, mag, dims = self._frequencies()
        # the MFMA kernel takes THIS layer's rows (another layer with as many heads may have planned tiles that this one
        # cannot use): bfloat16 queries then, float32 ones for the plain kernel
        mfma = ops.latent_attention_mfma_ok(batch.act_dtype, r, r + dr) and ("latent_parts", nh, self.window) in batch.shared
        qa = ops.latent_prepare(q_rows, qd[:, nq:nq + r + dr] if store else None, cache.rows if store else None,
                                batch.slot_mapping(cache.group) if store else None, self.c_norm, self.norm_eps, freq, mag, dims,
                                batch.positions, nh, dn, dr, r, torch.bfloat16 if mfma else torch.float32,
                                interleaved=bool(getattr(self.position, "interleaved", False)))
        gate_rows = qd[:, g0:g0 + nh] if self.has_gate else None
        qd = q_rows
        nq = nh * (dn + dr)
        D, ld = r + dr, qd.stride(0)
        library = mfma and T > ops.HEAD_PRODUCTS_MAX_ROWS and self.w_uk.dtype == torch.bfloat16
        # the unrotated query parts through the keys' expansion: qa[t, h, :r] = sum_d q[t, h, d] Wuk[h dn + d, :]
        if not dn:
            qa[:, :, :r].zero_()
        elif library:
            qa[:, :, :r].copy_(torch.bmm(qd[:, :nq].unflatten(1, (nh, dn + dr))[:, :, :dn].transpose(0, 1), self.w_uk.transpose(1, 2)).transpose(0, 1))
        elif mfma and self.w_uk.dtype == torch.bfloat16 and ops.head_products_ok(qd, ld, dn + dr, dn):
            ops.head_products(qd, ld, dn + dr, self.w_uk, qa, nh * D, D, T)
        else:
            ops.gemm_strided(qd, (dn + dr, ld, 1), self.w_uk, (r * dn, dn, 1), qa, (D, nh * D, 1), nh, T, r, dn)
        meta = attention_meta(batch, cache.group, nh)
        tiles, parts = None, 1
        if mfma:
            tiles = (batch.array("latent_tile_entry_%d" % nh), batch.array("latent_tile_row0_%d" % nh), batch.shared[("latent_tiles", nh)],
                     batch.shared[("latent_tile_rows", nh)])
            parts = batch.shared[("latent_parts", nh, self.window)]
        lat = ops.latent_attention(qa, cache.rows, cache.page_size, meta, self.sink, r, self.scale, self.window, x.dtype, tiles, parts)
        # the summed latents through the values' expansion: v[t, h, e] = sum_j lat[t, h, j] Wuv[h dv + e, j]
        if library and self.w_uv.dtype == torch.bfloat16:
            v = torch.bmm(lat.transpose(0, 1), self.w_uv.transpose(1, 2)).transpose(0, 1).reshape(T, nh * dv)
        else:
            v = torch.empty((T, nh * dv), dtype=x.dtype, device=x.device)
            if self.w_uv.dtype == torch.bfloat16 and ops.head_products_ok(lat, nh * r, r, r):
                ops.head_products(lat, nh * r, r, self.w_uv, v, nh * dv, dv, T)
            else:
                ops.gemm_strided(lat, (r, nh * r, 1), self.w_uv, (dv * r, r, 1), v, (dv, nh * dv, 1), nh, T, dv, r)
        if gate_rows is not None:
            ops.sigmoid_gate(v, gate_rows, per=dv)
        return ops.linear_few(v, self.w_o, self.w_o_tiled)
