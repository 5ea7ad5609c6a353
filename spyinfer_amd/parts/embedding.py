"""Token embedding and output head.  h[t] = E[id[t]] with no scaling
(src/models/qwen3.hpp:114-119); logits = norm(h) . W^T for the asked rows only, W = E when the
model ties them (src/models/qwen3.hpp:46, 283-301)."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Part


class TokenEmbedding(Part):
    def __init__(self, vocab_size: int, hidden_size: int, scale: float = 1.0, suffix: str = ".weight"):
        """``scale``: h[t] = E[id[t]] * scale (a tied head still reads the table as it is stored)."""
        self.vocab_size, self.hidden_size = vocab_size, hidden_size
        self.scale, self.suffix = float(scale), suffix
        self.weight = None

    def weight_specs(self, prefix):
        return [WeightSpec(prefix + self.suffix, (self.vocab_size, self.hidden_size))]

    def bind(self, prefix, weights):
        self.weight = weights[prefix + self.suffix]

    def capturable(self, batch):
        return True

    def forward(self, ids):
        return ops.embedding(ids, self.weight, self.scale)

    def forward_for(self, ids, norm, act_dtype):
        """(stream, pending) with the input of ``norm`` prepared where few rows and a foldable norm allow it."""
        fold = norm.foldable(act_dtype) if norm is not None else None
        if fold is None or self.scale != 1.0 or not ops.fused_decode_ok(ids.shape[0], act_dtype):
            return ops.embedding(ids, self.weight, self.scale), None
        return ops.embedding_scaled(ids, self.weight, fold[0], fold[1], norm)


class LMHead(Part):
    def __init__(self, vocab_size: int, hidden_size: int, tied_to: TokenEmbedding = None, fold_rows: int = 64, suffix: str = ".weight",
                 scale: float = 1.0, softcap: float = 0.0):
        """``fold_rows``: most rows for which the head runs as a decode product with the final norm folded in.  Above,
        the library's product after a norm kernel is faster for a large matrix (measured with 151936 x 4096: 235 / 246 /
        253 / 267 us at 24 / 32 / 48 / 64 rows against the library's 263 / 270 / 258 / 268 and a norm kernel of 6, but
        281 / 288 / 367 against 274 / 280 / 293 at 80 / 96 / 128).  ``scale``, ``softcap``: the logits are multiplied by
        ``scale`` and then, with a cap > 0, become cap tanh(logit / cap), in float32 and in place."""
        self.scale, self.softcap = float(scale), float(softcap)
        self.vocab_size, self.hidden_size, self.tied_to = vocab_size, hidden_size, tied_to
        self.fold_rows = fold_rows
        self.suffix = suffix
        self.weight = None

    def weight_specs(self, prefix):
        if self.tied_to is not None:
            # a tied checkpoint may store the head again; it is not read (src/models/qwen3.hpp:46)
            return [WeightSpec(prefix + self.suffix, (self.vocab_size, self.hidden_size), optional=True)]
        return [WeightSpec(prefix + self.suffix, (self.vocab_size, self.hidden_size))]

    def bind(self, prefix, weights):
        if self.tied_to is not None:
            self.weight, self.weight_tiled = ops.weight_forms(self.tied_to.weight, keep_rows=True)   # the table's rows are looked up
        else:
            self.weight, self.weight_tiled = ops.weight_forms(weights.pop(prefix + self.suffix))

    def capturable(self, batch):
        return True

    def can_fold(self, batch):
        # without the matrix's rows the library's product would have them restored first (more bytes than the product
        # itself reads): the folded product stands as far as it is built
        rows = ops.FUSED_DECODE_MAX_ROWS if isinstance(self.weight, ops.TiledOnly) else self.fold_rows
        return ops.fused_decode_ok(batch.T, batch.act_dtype, self.weight_tiled, max_rows=rows)

    def logits(self, resid, pending, final_norm, batch, out=None):
        """The end of a forward pass: ``final_norm`` of the stream (``pending`` as a block leaves it: None, an addend
        or the prepared input of a norm) at the batch's wanted rows, then the head."""
        if isinstance(pending, ops.ScaledInput):
            if pending.norm is final_norm and batch.all_rows_wanted and self.can_fold(batch):
                return self.forward(pending, out)
            pending = None                       # the stream is complete
        return self.forward(final_norm.add_norm(resid, pending, batch.act_dtype, batch.logit_rows), out)

    def forward(self, normed, out=None):
        """float32 logits [rows, vocab]; written into ``out`` if the caller brings a tensor of that shape."""
        logits = self._product(normed, out)
        if self.scale != 1.0 or self.softcap > 0.0:
            ops.scale_cap(logits, self.scale, self.softcap)
        return logits

    def _product(self, normed, out=None):
        if isinstance(normed, ops.ScaledInput):
            return ops.decode_linear(normed, self.weight_tiled, torch.float32, out)
        if normed.shape[0] <= self.fold_rows:
            return ops.linear_few(normed, self.weight, self.weight_tiled, torch.float32, out)      # the decode products, without a folded norm
        return ops.linear(normed, self.weight, torch.float32, tiled=self.weight_tiled, out=out)


class PairHashEmbedding(TokenEmbedding):
    """h[t] = E[id[t]] + B[row], row = (previous id * mul_prev + id[t] * mul_cur) mod buckets: a second table indexed by
    a hash of the token and the one before it; a request's first token takes the table's last row (number ``buckets``).
    The previous token of an entry's first token is part of the request's state: a slot of one int32
    (``cache_spec``), which the step leaves at the entry's last token.  Without a pair table (``buckets`` = 0) it is a
    plain embedding."""

    def __init__(self, vocab_size: int, hidden_size: int, buckets: int = 0, mul_prev: int = 0, mul_cur: int = 0,
                 names=("embed", "bigram")):
        super().__init__(vocab_size, hidden_size)
        self.buckets, self.mul_prev, self.mul_cur, self.names = int(buckets), int(mul_prev), int(mul_cur), names
        self.pair = None

    def weight_specs(self, prefix):
        e, b = (prefix + n for n in self.names)
        specs = [WeightSpec(e, (self.vocab_size, self.hidden_size))]
        if self.buckets:
            specs.append(WeightSpec(b, (self.buckets + 1, self.hidden_size)))
        return specs

    def bind(self, prefix, weights):
        e, b = (prefix + n for n in self.names)
        self.weight = weights[e]
        if self.buckets:
            self.pair = weights[b]
            if self.pair.dtype != self.weight.dtype:
                self.weight, self.pair = self.weight.float(), self.pair.float()

    def cache_spec(self):
        from ..cache.spec import FixedState
        return FixedState((1,), "int32") if self.buckets else None

    def forward_step(self, batch, cache):
        """(stream float32 [T, H], its copy in the activation dtype or None) for the step's tokens."""
        last = cache.state.view(-1) if cache is not None else None
        return ops.pair_embedding(batch.token_ids, self.weight, self.pair, self.buckets, self.mul_prev, self.mul_cur,
                                  batch.positions, batch.array("token_entry"), batch.array("cu_q"), batch.array("slot_ids"),
                                  last, batch.act_dtype)
