"""A decoder as data: an embedding, a list of layers (blocks of parts), the
order in which they run, a final norm and an output head.

The run order is a list of ``LayerCall``s.  It may name a layer twice (its
weights are used again, each call with a cache of its own) or let a call read
the cache that another call writes (``cache`` = that call's cache id,
``store=False``).  A call may stand at the start of a walk over a run of layers
(``enter`` = the walk's number): the model's ``pass_entry`` part then says what
meets the stream there.  By default layer i runs once with cache i, as in the
reference (src/models/qwen3.hpp:122-278).
"""
from __future__ import annotations

from typing import Dict, List, NamedTuple, Optional, Sequence

import torch

from ..kernels import ops
from ..parts.base import Block, Norm, PositionEncoding
from ..parts.block import stream_copy
from ..parts.embedding import LMHead, TokenEmbedding
from ..weights.loader import WeightSpec


class LayerCall(NamedTuple):
    layer: int
    cache: Optional[int] = None   # cache id; None = the call has no cache of its own kind
    store: bool = True            # False: read cache ``cache`` without writing
    enter: Optional[int] = None   # the number of the walk over a run of layers that begins with this call (``pass_entry``)


class DecoderModel:
    def __init__(self, config, embed: TokenEmbedding, position: Optional[PositionEncoding], layers: Sequence[Block],
                 final_norm: Norm, lm_head: LMHead, schedule: Optional[Sequence[LayerCall]] = None,
                 names: Dict[str, str] = None, max_positions: int = 0, pass_entry=None):
        """``pass_entry``: a part (``parts.block.PassEntry``) for run orders that walk a run of layers several times: the
        calls with ``enter`` set hand it what the block before left pending, and the embedding output if it asks for it."""
        self.config = config
        self.pass_entry = pass_entry
        self.embed, self.position, self.layers = embed, position, list(layers)
        self.final_norm, self.lm_head = final_norm, lm_head
        self.schedule = list(schedule) if schedule is not None else [LayerCall(i, i) for i in range(len(self.layers))]
        n = dict(embed="model.embed_tokens", position="model.position", layers="model.layers.%d", final_norm="model.norm",
                 lm_head="lm_head", pass_entry="model.pass_entry")
        n.update(names or {})
        self.names = n
        self.max_positions = max_positions
        self.vocab_size = lm_head.vocab_size
        for call in self.schedule:
            if not (0 <= call.layer < len(self.layers)):
                raise ValueError("the run order names layer %d of %d" % (call.layer, len(self.layers)))
            if call.enter is not None and pass_entry is None:
                raise ValueError("the run order has a walk's start, the model no part for it")
        self.cache_specs()  # validates the run order

    # ---- weights ---------------------------------------------------------
    def weight_specs(self) -> List[WeightSpec]:
        specs = list(self.embed.weight_specs(self.names["embed"]))
        if self.position is not None:
            specs += self.position.weight_specs(self.names["position"])
        for i, layer in enumerate(self.layers):
            specs += layer.weight_specs(self.names["layers"] % i)
        specs += self.final_norm.weight_specs(self.names["final_norm"])
        specs += self.lm_head.weight_specs(self.names["lm_head"])
        if self.pass_entry is not None:
            specs += self.pass_entry.weight_specs(self.names["pass_entry"])
        return specs

    def bind(self, weights: Dict[str, torch.Tensor], device) -> None:
        self.embed.bind(self.names["embed"], weights)
        if self.position is not None:
            self.position.bind(self.names["position"], weights)
            self.position.prepare(device, self.max_positions)
        for i, layer in enumerate(self.layers):
            layer.bind(self.names["layers"] % i, weights)
        self.final_norm.bind(self.names["final_norm"], weights)
        self.lm_head.bind(self.names["lm_head"], weights)
        if self.pass_entry is not None:
            self.pass_entry.bind(self.names["pass_entry"], weights)

    # ---- cache -----------------------------------------------------------
    def cache_specs(self) -> List[Optional[object]]:
        """Need of every cache id, taken from the call that writes it.  A mixer made of several (its ``cache_spec`` is a
        list) has the call's cache id for the first of them and further ids, behind the calls' own, for the others; its
        ``forward`` is handed the layer caches as a tuple in the list's order."""
        ids = [c.cache for c in self.schedule if c.cache is not None]
        specs: List[Optional[object]] = [None] * (max(ids) + 1 if ids else 0)
        writers, several = {}, {}
        for call in self.schedule:
            if call.cache is None or not call.store:
                continue
            if call.cache in writers:
                raise ValueError("cache %d is written by two calls of the run order" % call.cache)
            writers[call.cache] = call
            need = self.layers[call.layer].mixer.cache_spec()
            if isinstance(need, (list, tuple)):
                several[call.cache] = list(need)
                need = need[0] if need else None
            specs[call.cache] = need
        for call in self.schedule:
            if call.cache is not None and not call.store:
                if call.cache not in writers:
                    raise ValueError("a call reads cache %d that no call writes" % call.cache)
                need = self.layers[call.layer].mixer.cache_spec()
                if (list(need) != several.get(call.cache)) if isinstance(need, (list, tuple)) else (call.cache in several or need != specs[call.cache]):
                    raise ValueError("layer %d reads cache %d of another shape" % (call.layer, call.cache))
        #: cache id of a call -> the ids of all caches of its mixer, for mixers made of several
        self.cache_parts = {}
        for cid in sorted(several):
            self.cache_parts[cid] = [cid] + list(range(len(specs), len(specs) + len(several[cid]) - 1))
            specs += several[cid][1:]
        # an embedding that keeps something per request (the token before, say) has the cache id after the layers'
        own = getattr(self.embed, "cache_spec", None)
        self.embed_cache = None
        if own is not None and own() is not None:
            self.embed_cache = len(specs)
            specs.append(own())
        return specs

    # ---- step ------------------------------------------------------------
    def plan(self, batch) -> None:
        for call in self.schedule:
            self.layers[call.layer].mixer.plan(batch)

    def plan_ints(self, entries: int) -> int:
        """Most int32 values that the mixers' plans add to a step of ``entries`` single tokens (``Mixer.plan_arrays``)."""
        arrays = {}
        for call in self.schedule:
            arrays.update(self.layers[call.layer].mixer.plan_arrays(entries))
        return sum(arrays.values()) + 4 * len(arrays)

    def capturable(self, batch) -> bool:
        """Whether this step may be recorded in a HIP graph: every part that runs in it says so (``Part.capturable``)."""
        parts = [self.embed, self.final_norm, self.lm_head] + [self.layers[i] for i in sorted({c.layer for c in self.schedule})]
        if self.pass_entry is not None:
            parts.append(self.pass_entry)
        if self.position is not None:
            parts.append(self.position)
        return all(p.capturable(batch) for p in parts)

    def forward(self, batch, storage, logits_out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Runs the batch's tokens through all calls of the run order; float32 logits [R, vocab]
        at the batch's wanted rows (in ``logits_out`` if the caller brings a tensor of that shape)."""
        calls = self.schedule
        entry = [self.layers[c.layer].entry_norm() for c in calls] + [self.final_norm]
        if hasattr(self.embed, "forward_step"):
            # an embedding that reads more of the step than the token ids (and may keep state per request)
            resid, copy = self.embed.forward_step(batch, storage.layer(self.embed_cache) if self.embed_cache is not None else None)
            stream_copy(batch, resid, copy)
            pending = None
        elif self.position is None or type(self.position).on_embeddings is PositionEncoding.on_embeddings:
            resid, pending = self.embed.forward_for(batch.token_ids, entry[0], batch.act_dtype)
        else:
            resid, pending = self.position.on_embeddings(self.embed.forward(batch.token_ids), batch), None
        embedded = None
        if self.pass_entry is not None and self.pass_entry.needs_embedding() and any(c.enter for c in calls):
            # the embedding output meets the stream again later, and the stream is summed in place: a copy
            if pending is not None and not isinstance(pending, ops.ScaledInput):
                raise ValueError("the embedding left an addend pending: its output is not in the stream yet")
            embedded = resid.clone()
        for i, call in enumerate(calls):
            if call.enter is not None:
                pending = self.pass_entry.join(pending, embedded, call.enter)
            cache = storage.layer(call.cache) if call.cache is not None else None
            if call.cache in self.cache_parts:
                cache = tuple(storage.layer(c) for c in self.cache_parts[call.cache])
            resid, pending = self.layers[call.layer].forward(resid, pending, batch, cache, call.store, next_norm=entry[i + 1])
        if batch.R == 0:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=resid.device) if logits_out is None else logits_out
        return self.lm_head.logits(resid, pending, self.final_norm, batch, logits_out)
