"""Grouped-query attention over the paged cache.

Per step: fused q/k/v projection; per-head RMS norm of q and k (optional;
before the rotation, src/models/qwen3.hpp:160-194); rotation; keys and values
of all tokens of the step written to their pages before any query reads
(src/backends/cpu/cpu_attention.cpp:61-68); then every query reads its keys
through its request's block table with the causal mask ``key <= position``
(:98-111), scale 1/sqrt(d) after the dot product (:59, :110), kv head
``h * n_kv / n_q`` (:96); output projection.  One meaning for whole prompts,
portions and single tokens.  ``window`` keeps only the last ``window`` keys.

Options beside the reference's arrangement: biases on the q, k and v projections; a value size other than the
key size (the smaller of the two is padded with zero rows when the weights are bound, so that one head size runs
through cache and kernels); a sigmoid gate on the concatenated heads, projected from the mixer's input beside
q, k and v; a rotation whose angles are formed in the kernel from the encoding's frequencies (no table and no
position limit: encodings with rescaled frequencies, with or without a factor on cos and sin); values divided by their
root mean square per head before they are stored; scores capped by cap tanh(score / cap) after the scale; queries
multiplied by a temperature that grows with the logarithm of the position; a penalty r1_h ln(1 + r2_h (i - j)) on the
distance, taken off the (capped) score; a softmax whose denominator holds a one (a sink of score 0 without a value); the
gate as one number per head instead of one per value.
"""
from __future__ import annotations

import math
from typing import Optional

import numpy as np
import torch

from ..cache.spec import PagedKV
from ..kernels import key_pieces, ops
from ..weights.loader import WeightSpec
from .base import Mixer, PositionEncoding


ROWS_PER_TILE = 16        # rows of (token, head-in-group) pairs in a small attention tile
BIG_MIN_ROWS = 64         # entries with at least this many rows go to the prefill kernel


def plan_attention_tiles(batch, group_size: int, big_rows: int = 0, key_parts: bool = True) -> None:
    """Adds to the step's arrays the tiles over each entry's rows (token-major, head-in-group minor) for a query-head
    group of ``group_size``: entries with at least BIG_MIN_ROWS rows are cut into tiles of ``big_rows`` rows (the
    LDS-sharing prefill kernel; 0: never), the others into 16-row tiles (one block of waves each).  Once per step,
    group size and tile size.  ``key_parts``: the caller's launches take the number of key parts from the longest
    request (False: its keys are cut another way, ``plan_decode_pieces``)."""
    if key_parts:
        # the 16-row tiles' keys are split into a number of parts that follows the longest request: a launch shape
        batch.add_graph_key("attention_key_parts", ops.key_parts_for(batch.max_kv_len))
    note = ("attention_tiles", group_size, big_rows)
    if note in batch.shared:
        return
    S, lens = batch.S, batch.lens
    rows = lens.astype(np.int64) * group_size
    big = (rows >= BIG_MIN_ROWS) & bool(big_rows)
    counts = {}
    for kind, size, mask in (("small", ROWS_PER_TILE, ~big), ("big", max(big_rows, 1), big)):
        ntiles = np.where(mask, (rows + size - 1) // size, 0)
        tile_entry = np.repeat(np.arange(S, dtype=np.int32), ntiles)
        first = np.zeros(S + 1, dtype=np.int64)
        np.cumsum(ntiles, out=first[1:])
        tile_row0 = ((np.arange(int(first[-1]), dtype=np.int64) - first[:-1][tile_entry]) * size).astype(np.int32)
        if kind == "big" and tile_entry.shape[0] > 2:
            # the prefill kernel gives a block the tiles b and n - 1 - b: sorted by the keys they read, blocks are even
            pos0 = batch.host_array("pos0")[tile_entry].astype(np.int64)
            last_tok = np.minimum(lens[tile_entry].astype(np.int64), (tile_row0.astype(np.int64) + size + group_size - 1) // group_size)
            order = np.argsort(-(pos0 + last_tok), kind="stable")
            tile_entry, tile_row0 = tile_entry[order], tile_row0[order]
        counts[kind] = int(first[-1])
        batch.add_array("tile_entry_%s_%d_%d" % (kind, group_size, big_rows), tile_entry)
        batch.add_array("tile_row0_%s_%d_%d" % (kind, group_size, big_rows), tile_row0)
    batch.shared[note] = counts


def plan_decode_pieces(batch, n_kv: int, window: int, head_dim: int) -> None:
    """Adds to the arrays of a step of single tokens its keys cut into pieces of even size (``key_pieces.decode_pieces``), for
    layers of ``n_kv`` kv heads of ``head_dim`` and this window.  The array's length follows the numbers of entries and
    heads alone."""
    note = ("decode_pieces", n_kv, window, head_dim)
    if note not in batch.shared:
        batch.add_array("decode_pieces_%d_%d_%d" % note[1:], key_pieces.decode_pieces(batch.host_array("kv_len"), n_kv, window, head_dim=head_dim))
        batch.shared[note] = True


def attention_meta(batch, group: int, group_size: int, big_rows: int = 0) -> ops.AttentionMeta:
    """The step's description for the attention kernels, from the batch's arrays on the device (one object per step,
    cache group, group size and tile size)."""
    note = ("attention_meta", group, group_size, big_rows)
    meta = batch.shared.get(note)
    if meta is None:
        tiles = None
        counts = batch.shared.get(("attention_tiles", group_size, big_rows))
        if counts is not None:
            tiles = {kind: (batch.array("tile_entry_%s_%d_%d" % (kind, group_size, big_rows)),
                            batch.array("tile_row0_%s_%d_%d" % (kind, group_size, big_rows)), n) for kind, n in counts.items()}
        pieces = {key[1:]: batch.array("decode_pieces_%d_%d_%d" % key[1:]).view(-1, key_pieces.PIECE_RECORD)
                  for key in batch.shared if isinstance(key, tuple) and key[0] == "decode_pieces"}
        meta = ops.AttentionMeta(batch.array("cu_q"), batch.array("pos0"), batch.array("kv_len"), batch.block_table(group),
                                 batch.array("token_entry"), batch.array("positions"), batch.S, batch.T, batch.max_blocks[group],
                                 batch.max_kv_len, batch.max_q_len, tiles, group_size, fixed_shape=batch.fixed_shape,
                                 big_rows=big_rows or 128, pieces=pieces)
        batch.shared[note] = meta
    return meta


class PagedAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: Optional[PositionEncoding], qk_norm_eps: Optional[float] = None,
                 window: Optional[int] = None, scale: Optional[float] = None, fold_rows: Optional[int] = None,
                 value_dim: Optional[int] = None, bias: bool = False, gate: bool = False, names: Optional[dict] = None,
                 softcap: float = 0.0, value_norm_eps: Optional[float] = None, query_temperature=None, distance_penalty: bool = False,
                 zero_sink: bool = False):
        """``fold_rows``: most rows of a step whose products here run with the norms and the residual sum folded in
        (None: ``ops.default_fold_rows`` of this part's matrices).  ``value_dim``: size of a value head (None: ``head_dim``).
        ``bias``: q, k and v have biases.  ``gate``: the heads' results are multiplied by sigmoid(Wg x) before the output
        projection.  ``names``: tensor names behind the prefix for q, k, v, o, g, q_norm, k_norm and the biases' suffix
        ``bias``.  ``softcap`` > 0: score = softcap tanh(q . k scale / softcap).  ``value_norm_eps``: every value head is
        divided by sqrt(mean(v^2) + eps) over its ``value_dim`` values (no weight) and cached so.  ``gate`` "head": the
        gate is one number per head (a matrix [heads, hidden]) instead of one per value.  ``query_temperature`` = (coef,
        every): the query at position p is multiplied by 1 + coef ln(floor((p + 1) / every) + 1).  ``distance_penalty``:
        two numbers per head (tensors ``r1``, ``r2`` [heads]); the score of a key x positions back is lowered by
        r1 ln(1 + r2 x), after the cap.  ``zero_sink``: p_j = e^(s_j) / (1 + sum e^(s_j))."""
        if num_heads % num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.key_dim, self.value_dim = head_dim, head_dim if value_dim is None else value_dim
        # one head size for cache and kernels: where key and value sizes differ, the larger, in whole MFMA tiles
        self.head_dim = head_dim if self.value_dim == head_dim else -(-max(head_dim, self.value_dim) // 16) * 16
        self.has_bias, self.has_gate = bool(bias), bool(gate)
        self.gate_per_head = gate == "head"
        self.query_temperature = None if query_temperature is None else (float(query_temperature[0]), int(query_temperature[1]))
        self.has_distance, self.zero_sink = bool(distance_penalty), bool(zero_sink)
        self.distance = None
        self.names = dict(q=".q_proj.weight", k=".k_proj.weight", v=".v_proj.weight", o=".o_proj.weight", g=".g_proj.weight",
                          q_norm=".q_norm.weight", k_norm=".k_norm.weight", bias=".bias", r1=".r1", r2=".r2")
        self.names.update(names or {})
        self.b_qkv = None
        self.position = position
        self.qk_norm_eps = qk_norm_eps
        self.window = window
        self.scale = 1.0 / math.sqrt(head_dim) if scale is None else float(scale)
        self.fold_rows = fold_rows
        self.softcap = float(softcap or 0.0)
        self.value_norm_eps = None if value_norm_eps is None else float(value_norm_eps)
        self.w_qkv = self.w_o = self.q_norm = self.k_norm = self.w_qkv_tiled = self.w_o_tiled = None

    # ---- weights ---------------------------------------------------------
    def weight_specs(self, prefix):
        H, nq, nkv, dk, dv, n = self.hidden_size, self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim, self.names
        specs = [WeightSpec(prefix + n["q"], (nq * dk, H)), WeightSpec(prefix + n["k"], (nkv * dk, H)),
                 WeightSpec(prefix + n["v"], (nkv * dv, H)), WeightSpec(prefix + n["o"], (H, nq * dv))]
        if self.has_bias:
            specs += [WeightSpec(prefix + n["q"] + n["bias"], (nq * dk,), "bias"), WeightSpec(prefix + n["k"] + n["bias"], (nkv * dk,), "bias"),
                      WeightSpec(prefix + n["v"] + n["bias"], (nkv * dv,), "bias")]
        if self.has_gate:
            specs.append(WeightSpec(prefix + n["g"], (nq if self.gate_per_head else nq * dv, H)))
        if self.has_distance:
            specs += [WeightSpec(prefix + n["r1"], (nq,), "bias"), WeightSpec(prefix + n["r2"], (nq,), "norm")]
        if self.qk_norm_eps is not None:
            specs += [WeightSpec(prefix + n["q_norm"], (dk,), "norm"), WeightSpec(prefix + n["k_norm"], (dk,), "norm")]
        return specs

    def _padded(self, t: torch.Tensor, heads: int, size: int) -> torch.Tensor:
        """Rows (or entries) [heads * size, ...] -> [heads * head_dim, ...], every head filled up with zeros."""
        d = self.head_dim
        if size == d:
            return t
        out = torch.zeros((heads, d) + tuple(t.shape[1:]), dtype=t.dtype, device=t.device)
        out[:, :size] = t.view((heads, size) + tuple(t.shape[1:]))
        return out.view((heads * d,) + tuple(t.shape[1:]))

    def bind(self, prefix, weights):
        # the matrices leave the caller's dictionary here, so that they are freed once they are fused: binding a
        # model never holds the separate matrices, the fused one and its tiled copy of all layers at once
        n, nq, nkv, dk, dv = self.names, self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        mats = [weights.pop(prefix + n[c]) for c in "qkv"] + ([weights.pop(prefix + n["g"])] if self.has_gate else [])
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        if self.has_gate and self.gate_per_head:
            # one row per head; zero rows behind them bring the fused matrix to whole tiles of 16 rows
            fill = -(nq + (nq + 2 * nkv) * self.head_dim) % 16
            gate_rows = torch.cat([mats[3], torch.zeros((fill, mats[3].shape[1]), dtype=mats[3].dtype, device=mats[3].device)]) if fill else mats[3]
            mats = [self._padded(m, heads, size) for m, heads, size in zip(mats[:3], (nq, nkv, nkv), (dk, dk, dv))] + [gate_rows]
        else:
            mats = [self._padded(m, heads, size) for m, heads, size in zip(mats, (nq, nkv, nkv, nq), (dk, dk, dv, dv))]
        # one product for q, k and v (and the gate): rows [q heads | k heads | v heads | gate]
        self.w_qkv = torch.cat(mats, dim=0).contiguous()
        del mats
        self.w_qkv, self.w_qkv_tiled = ops.weight_forms(self.w_qkv)
        w_o = weights.pop(prefix + n["o"])
        if dv != self.head_dim:
            w_o = self._padded(w_o.t().contiguous(), nq, dv).t().contiguous()
        self.w_o, self.w_o_tiled = ops.weight_forms(w_o)
        if self.has_bias:
            b = [weights[prefix + n[c] + n["bias"]] for c in "qkv"]
            if len({t.dtype for t in b}) > 1:
                b = [t.float() for t in b]
            self.b_qkv = torch.cat([self._padded(t, heads, size) for t, heads, size in zip(b, (nq, nkv, nkv), (dk, dk, dv))]).contiguous()
        if self.has_distance:
            # the penalty's numbers enter the scores, which are float32: [2, heads]
            self.distance = torch.stack([weights[prefix + n["r1"]].float(), weights[prefix + n["r2"]].float()]).contiguous()
        if self.qk_norm_eps is not None:
            if dk != self.head_dim:
                raise ValueError("per-head norms of q and k with a value size other than the key size are not implemented")
            self.q_norm, self.k_norm = weights[prefix + n["q_norm"]], weights[prefix + n["k_norm"]]
            if self.q_norm.dtype != self.k_norm.dtype:
                self.q_norm, self.k_norm = self.q_norm.float(), self.k_norm.float()
        if self.position is not None and not self._plain_projections():
            self.position.prepare(self.w_o.device, 0)

    # ---- cache -----------------------------------------------------------
    def cache_spec(self):
        return PagedKV(self.num_kv_heads, self.head_dim, self.window)

    def plan(self, batch) -> None:
        # a step of single tokens that the fused kernel will take has its keys cut into even pieces on the host
        pieces = ops.decode_pieces_ok(batch.S, batch.T, batch.act_dtype, self.num_kv_heads, self.head_dim) and self._rotated_whole()
        plan_attention_tiles(batch, self.num_heads // self.num_kv_heads, self._big_rows(batch, batch.page_size), key_parts=not pieces)
        if pieces:
            plan_decode_pieces(batch, self.num_kv_heads, int(self.window or 0), self.head_dim)

    def plan_arrays(self, entries):
        G = self.num_heads // self.num_kv_heads
        out = {"tile_entry_small_%d" % G: entries, "tile_row0_small_%d" % G: entries}
        if ops.decode_pieces_ok(entries, entries, torch.bfloat16, self.num_kv_heads, self.head_dim):
            out["decode_pieces_%d_%d_%d" % (self.num_kv_heads, int(self.window or 0), self.head_dim)] = \
                key_pieces.decode_pieces_capacity(entries, self.num_kv_heads) * key_pieces.PIECE_RECORD
        return out

    def _plain_projections(self) -> bool:
        """No bias, no gate and a rotation by table: the arrangement that the fused kernels and the folded products know.
        Otherwise one kernel adds the biases, rotates by angles that it forms itself from the encoding's frequencies (an
        encoding with rescaled frequencies has no table) and stores."""
        return not (self.has_bias or self.has_gate or self.softcap or self.value_norm_eps is not None
                    or self.query_temperature is not None or self.has_distance or self.zero_sink
                    or (self.position is not None and getattr(self.position, "scaling", None) is not None))

    def _rotated_whole(self) -> bool:
        """The head is rotated whole or not at all, and the group is one tile: what the fused kernel takes."""
        if not self._plain_projections():
            return False
        rot = self.position.rotary() if self.position is not None else None
        return (rot is None or rot[2] in (0, self.head_dim)) and self.num_heads // self.num_kv_heads <= 16

    def _big_rows(self, batch, page_size: int) -> int:
        """Rows of the tiles for this step's entries with many rows; 0 if the prefill kernel does not take this head
        size or page."""
        if not ops.prefill_attention_ok(self.head_dim, page_size):
            return 0
        note = ("attention_big_rows", self.num_heads, self.num_kv_heads, self.head_dim)
        if note not in batch.shared:
            rows = batch.lens.astype(np.int64) * (self.num_heads // self.num_kv_heads)
            batch.shared[note] = ops.prefill_tile_rows(self.head_dim, rows[rows >= BIG_MIN_ROWS], self.num_kv_heads)
        return batch.shared[note]

    # ---- step ------------------------------------------------------------
    def capturable(self, batch):
        # everything a step changes is read from the batch's device arrays; the one launch shape that follows the
        # requests' lengths, the number of key parts, is in the graph's key (plan_attention_tiles)
        return self.position is None or self.position.capturable(batch)

    def can_fold(self, batch):
        # (beyond 64 rows the products take their inputs in operand order only: the attention must hand its result over so)
        if not self._plain_projections():
            return False
        if batch.T > 64 and not ops.attention_hands_over_operand_rows(batch.act_dtype, self.num_heads, self.head_dim, batch.page_size):
            return False
        return ops.fused_decode_ok(batch.T, batch.act_dtype, self.w_qkv_tiled, self.w_o_tiled, max_rows=self.fold_rows)

    def _attend(self, x, batch, cache, store, for_product=False):
        nq, nkv, d = self.num_heads, self.num_kv_heads, self.head_dim
        if isinstance(x, ops.ScaledInput):
            qkv = ops.decode_linear(x, self.w_qkv_tiled)
        elif not self._plain_projections():
            qkv = ops.linear_few(x, self.w_qkv, self.w_qkv_tiled)       # (no folded path here: the decode products up to 64 rows)
        else:
            qkv = ops.linear(x, self.w_qkv, tiled=self.w_qkv_tiled)
        meta = attention_meta(batch, cache.group, nq // nkv, self._big_rows(batch, cache.page_size))
        if not self._plain_projections():
            # biases, rotation and store in one kernel that reads q, k and v out of the wider product; the gate's rows,
            # which lie behind them, are multiplied into the heads' results
            if self.qk_norm_eps is not None:
                raise ValueError("per-head norms of q and k beside biases, a gate or rescaled frequencies are not implemented")
            freq, mag, rdim = None, 1.0, 0
            if self.position is not None:
                freq, mag, rdim = self.position.frequencies()
            slots = batch.slot_mapping(cache.group) if store else None
            vnorm = None if self.value_norm_eps is None else (self.value_norm_eps, self.value_dim)
            q = ops.bias_rope_store(qkv, nq, nkv, d, self.b_qkv, freq, rdim, batch.positions, cache.k, cache.v, cache.page_size, slots,
                                    mag=mag, value_norm=vnorm, query_temperature=self.query_temperature)
            out = ops.paged_attention(q, cache.k, cache.v, cache.page_size, meta, nq, nkv, d, self.scale, self.window, softcap=self.softcap,
                                      distance=self.distance, zero_sink=self.zero_sink)
            if self.has_gate and self.gate_per_head:
                g0 = (nq + 2 * nkv) * d
                ops.sigmoid_gate(out, qkv[:, g0:g0 + nq], per=d)
            elif self.has_gate:
                ops.sigmoid_gate(out, qkv[:, (nq + 2 * nkv) * d:])
            return out
        rot = self.position.rotary() if self.position is not None else None
        cos, sin, rdim = rot if rot is not None else (None, None, 0)
        eps = self.qk_norm_eps if self.qk_norm_eps is not None else 0.0
        if ops.fused_attention_ok(qkv.dtype, meta, nq, nkv, d, cache.page_size, rdim, self.q_norm, self.k_norm):
            # single tokens only: the attention kernel norms, rotates and stores by itself
            raw = ops.RawQKV(qkv, self.q_norm, self.k_norm, eps, cos if rdim else None, sin if rdim else None, store)
            return ops.paged_attention(None, cache.k, cache.v, cache.page_size, meta, nq, nkv, d, self.scale, self.window, raw,
                                       for_product=for_product)
        slots = batch.slot_mapping(cache.group) if store else None
        q = ops.qk_norm_rope_store(qkv, nq, nkv, d, self.q_norm, self.k_norm, eps,
                                   cos, sin, rdim, batch.positions, cache.k, cache.v, cache.page_size, slots)
        return ops.paged_attention(q, cache.k, cache.v, cache.page_size, meta, nq, nkv, d, self.scale, self.window,
                                   for_product=for_product)

    def forward(self, x, batch, cache, store=True):
        if not self._plain_projections():
            return ops.linear_few(self._attend(x, batch, cache, store), self.w_o, self.w_o_tiled)
        return ops.linear(self._attend(x, batch, cache, store), self.w_o, tiled=self.w_o_tiled)

    def forward_into(self, x, batch, cache, store, resid, next_norm):
        weight, eps = next_norm.foldable(batch.act_dtype)
        return ops.decode_linear_residual(self._attend(x, batch, cache, store, for_product=True), self.w_o_tiled, resid, weight, eps,
                                          next_norm)
