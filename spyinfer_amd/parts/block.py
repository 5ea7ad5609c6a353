"""Pre-norm block: h += mixer(norm1(h)); h += ffn(norm2(h))  (src/models/qwen3.hpp:122-278).
The sums are carried as a pending addend and folded into the next norm's kernel."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Block, FeedForward, Mixer, Norm, Part


class ResultGate(Part):
    """What a sublayer's result is multiplied by before it meets the stream: ``mult`` * sigmoid(W n + b), element by
    element, n being the sublayer's input (the norm's output).  Tensors: the matrix under the prefix itself, the bias
    under ``<prefix>.b``."""

    def __init__(self, hidden_size: int, mult: float = 1.0, bias_suffix: str = ".b"):
        self.hidden_size, self.mult, self.bias_suffix = hidden_size, float(mult), bias_suffix
        self.w = self.w_tiled = self.bias = None

    def weight_specs(self, prefix):
        H = self.hidden_size
        return [WeightSpec(prefix, (H, H)), WeightSpec(prefix + self.bias_suffix, (H,), "bias")]

    def bind(self, prefix, weights):
        self.w, self.w_tiled = ops.weight_forms(weights.pop(prefix))
        self.bias = weights[prefix + self.bias_suffix]

    def capturable(self, batch):
        return True

    def apply(self, y, n):
        """y * mult * sigmoid(W n + b) as an addend whose gate the next norm's kernel applies (``ops.GatedAddend``)."""
        return ops.GatedAddend(y, ops.linear_few(n, self.w, self.w_tiled), self.bias, self.mult)


class PreNormBlock(Block):
    def __init__(self, norm1: Norm, mixer: Mixer, norm2: Norm = None, ffn: FeedForward = None,
                 names=("input_layernorm", "self_attn", "post_attention_layernorm", "mlp"), gates=None, gate_names=("rg1", "rg2")):
        """``ffn`` (with ``norm2``) may be absent.  ``gates``: None, or a pair of ``ResultGate`` (the second None without a
        feed-forward) that multiply the two sublayers' results, each reading its sublayer's input."""
        if (ffn is None) != (norm2 is None):
            raise ValueError("a feed-forward and its norm come together")
        self.norm1, self.mixer, self.norm2, self.ffn = norm1, mixer, norm2, ffn
        self.names = names
        self.gate1, self.gate2 = gates if gates is not None else (None, None)
        self.gate_names = gate_names

    def _parts(self, prefix):
        parts = list(zip((self.norm1, self.mixer, self.norm2, self.ffn), (prefix + "." + n for n in self.names)))
        parts += list(zip((self.gate1, self.gate2), (prefix + "." + n for n in self.gate_names)))
        return [(part, p) for part, p in parts if part is not None]

    def weight_specs(self, prefix):
        return [s for part, p in self._parts(prefix) for s in part.weight_specs(p)]

    def bind(self, prefix, weights):
        for part, p in self._parts(prefix):
            part.bind(p, weights)

    def entry_norm(self):
        return self.norm1

    def capturable(self, batch):
        return all(part.capturable(batch) for part, _ in self._parts(""))

    def forward(self, resid, pending, batch, cache, store=True, next_norm=None):
        act = batch.act_dtype
        ready = isinstance(pending, ops.ScaledInput)
        mine = ready and pending.norm is self.norm1
        plain = self.ffn is not None and self.gate1 is None and self.gate2 is None
        fold = plain and self.norm2.foldable(act) is not None and self.mixer.can_fold(batch) and self.ffn.can_fold(batch)
        if fold and not ops.folded_products_take(pending if mine else None, batch.T):
            # beyond 64 rows the folded products take an input in operand order only, which only the part before this
            # block can have prepared (another kind of block, a position encoding on the embeddings, parts that fold up
            # to fewer rows may not have): the plain path then
            fold = False
        if fold:
            # few rows: the sums go into the stream inside the products, the norms' scales into the products after them
            if mine:
                n1 = pending
            else:
                n1 = self.norm1.add_norm(resid, None if ready else pending, act)
            n2 = self.mixer.forward_into(n1, batch, cache, store, resid, self.norm2)
            if next_norm is not None and next_norm.foldable(act) is not None:
                return resid, self.ffn.forward_into(n2, batch, resid, next_norm)
            return resid, self.ffn.forward(n2, batch)
        n1 = self.norm1.add_norm(resid, None if ready else pending, act)
        a = self.mixer.forward(n1, batch, cache, store)
        if self.gate1 is not None:
            a = self.gate1.apply(a, n1)
        if self.ffn is None:
            return resid, a
        n2 = self.norm2.add_norm(resid, a, act)
        f = self.ffn.forward(n2, batch)
        return resid, (self.gate2.apply(f, n2) if self.gate2 is not None else f)


def stream_copy(batch, resid, copy=None):
    """The residual stream in the activation dtype, for the products that read the stream itself.  A kernel that has
    just written the stream leaves the copy here (``copy`` given); a reader asks for it (made now if nobody left one).
    With float32 activations the stream serves."""
    if resid.dtype == batch.act_dtype:
        return resid
    if copy is not None:
        batch.shared["stream_copy"] = (resid, copy)
        return copy
    held = batch.shared.get("stream_copy")
    if held is not None and held[0] is resid:
        return held[1]
    copy = resid.to(batch.act_dtype)
    batch.shared["stream_copy"] = (resid, copy)
    return copy


class DepthMix(Part):
    """What goes on to the next layer is a weighted sum of the results of all layers so far and of the embedding output:
    x = sum_j a[j] X_j, j = 0 .. index + 1, with X_0 the embedding output and X_(j+1) the result of layer j (before any
    such sum).  The step's results are kept in one float32 tensor [layers + 1, T, H], which the layers' results are
    written into where they arise."""

    def __init__(self, index: int, total: int, suffix: str = ""):
        """``index``: the layer call this mix follows (0-based); ``total``: calls in the model's run order."""
        self.index, self.total, self.suffix = index, total, suffix
        self.weight = None

    def weight_specs(self, prefix):
        return [WeightSpec(prefix + self.suffix, (self.index + 2,), "mix")]

    def bind(self, prefix, weights):
        self.weight = weights[prefix + self.suffix]

    def capturable(self, batch):
        return True

    def kept(self, batch, resid):
        """The step's kept results; made when the first layer asks, with the stream as it stands as X_0."""
        held = batch.shared.get("depth_kept")
        if held is None:
            held = torch.empty((self.total + 1,) + tuple(resid.shape), dtype=torch.float32, device=resid.device)
            held[0].copy_(resid)
            batch.shared["depth_kept"] = held
        return held

    def result_slot(self, batch, resid):
        """Where this layer's result X_(index+1) is to be written."""
        return self.kept(batch, resid)[self.index + 1]

    def operands(self, batch):
        """(kept results, how many of them are mixed, their weights): what the kernel that writes this layer's result
        needs to form the mix in the same pass (``Norm.add_normed``)."""
        return batch.shared["depth_kept"], self.index + 2, self.weight

    def mix(self, batch):
        """(the stream for the next layer, its copy in the activation dtype or None), as a pass of its own."""
        return ops.depth_mix(batch.shared["depth_kept"], self.index + 2, self.weight, batch.act_dtype)


class OutputNormBlock(Block):
    """h += norm1(mixer(h)); h += norm2(ffn(h)): the norm sits on a sublayer's OUTPUT, the sublayers read the stream
    itself.  ``ffn`` (with ``norm2``) may be absent.  ``depth``: a ``DepthMix`` after the layer."""

    def __init__(self, mixer: Mixer, norm1: Norm, ffn: FeedForward = None, norm2: Norm = None, depth: "DepthMix" = None,
                 names=("mix", "norm1", "mlp", "norm2", "dwa")):
        if (ffn is None) != (norm2 is None):
            raise ValueError("a feed-forward and its norm come together")
        self.mixer, self.norm1, self.ffn, self.norm2, self.depth = mixer, norm1, ffn, norm2, depth
        self.names = names

    def _parts(self, prefix):
        parts = zip((self.mixer, self.norm1, self.ffn, self.norm2, self.depth), (prefix + "." + n for n in self.names))
        return [(part, p) for part, p in parts if part is not None]

    def weight_specs(self, prefix):
        return [s for part, p in self._parts(prefix) for s in part.weight_specs(p)]

    def bind(self, prefix, weights):
        for part, p in self._parts(prefix):
            part.bind(p, weights)

    def capturable(self, batch):
        return all(part.capturable(batch) for part, _ in self._parts(""))

    def forward(self, resid, pending, batch, cache, store=True, next_norm=None):
        act = batch.act_dtype
        if isinstance(pending, ops.EntryAddends):
            pending.resolve(resid)
            pending = None
        if pending is not None and not isinstance(pending, ops.ScaledInput):
            for addend in (pending if isinstance(pending, (tuple, list)) else (pending,)):
                resid.add_((addend.resolve() if isinstance(addend, ops.GatedAddend) else addend).float())         # a block of another arrangement left an addend (or a pair of them)
        x = stream_copy(batch, resid)
        y = self.mixer.forward(x, batch, cache, store)
        out = self.depth.result_slot(batch, resid) if self.depth is not None else resid
        mix = self.depth.operands(batch) if self.depth is not None else None       # formed by the layer's last norm kernel
        last = self.ffn is None
        out, copy = self.norm1.add_normed(resid, y, out, act, mix if last else None)
        if not last:
            x = stream_copy(batch, out, copy)
            f = self.ffn.forward(x, batch)
            out, copy = self.norm2.add_normed(out, f, out, act, mix)
        stream_copy(batch, out, copy)
        return out, None


class PassEntry(Part):
    """What happens to the stream where a walk over a run of layers begins, when the run is walked several times with the
    same weights: before every walk but the first the embedding output (the stream as it was before the first layer) is
    added back, and before every walk, the first too, a learned vector of that walk.  Tensor: ``[walks, H]`` under the
    prefix.  Nothing is computed here: the addends go on to the norm that reads the stream next (``ops.EntryAddends``)."""

    def __init__(self, hidden_size: int, walks: int, add_embedding: bool = True):
        self.hidden_size, self.walks, self.add_embedding = hidden_size, int(walks), bool(add_embedding)
        self.steps = None

    def weight_specs(self, prefix):
        return [WeightSpec(prefix, (self.walks, self.hidden_size), "bias")]

    def bind(self, prefix, weights):
        self.steps = weights[prefix].float().contiguous()        # the stream is float32, and so is what is added to it

    def capturable(self, batch):
        return True

    def needs_embedding(self) -> bool:
        return self.add_embedding and self.walks > 1

    def join(self, pending, embedded, walk: int):
        """``pending`` as the block before left it; ``embedded``: the embedding output (float32 [T, H])."""
        if not 0 <= walk < self.walks:
            raise ValueError("walk %d of %d" % (walk, self.walks))
        return ops.EntryAddends(pending, embedded if (self.add_embedding and walk > 0) else None, self.steps[walk])


class ParallelBlock(Block):
    """h += mixer(n) + ffn(n) with n = norm(h): one norm, both sublayers read its output, and their results meet the
    stream together.  The two results go on as a pair of addends, which the next norm's kernel sums in float32 and adds
    to the stream in the pass that it makes anyway.  ``ffn`` may be absent.  ``norm2``: the feed-forward reads the stream
    through a norm of its own, h += mixer(norm(h)) + ffn(norm2(h)); both norms come out of one pass over the row."""

    def __init__(self, norm: Norm, mixer: Mixer, ffn: FeedForward = None, names=("norm1", "mix", "mlp", "norm2"), norm2: Norm = None):
        if norm2 is not None and ffn is None:
            norm2 = None                   # (a layer without a feed-forward has no use for its norm; it has no tensor either)
        self.norm, self.mixer, self.ffn, self.norm2 = norm, mixer, ffn, norm2
        self.names = tuple(names) + ("norm2",) * (4 - len(names))

    def _parts(self, prefix):
        parts = zip((self.norm, self.mixer, self.ffn, self.norm2), (prefix + "." + n for n in self.names))
        return [(part, p) for part, p in parts if part is not None]

    def weight_specs(self, prefix):
        return [s for part, p in self._parts(prefix) for s in part.weight_specs(p)]

    def bind(self, prefix, weights):
        for part, p in self._parts(prefix):
            part.bind(p, weights)

    def capturable(self, batch):
        return all(part.capturable(batch) for part, _ in self._parts(""))

    def forward(self, resid, pending, batch, cache, store=True, next_norm=None):
        act = batch.act_dtype
        pending = None if isinstance(pending, ops.ScaledInput) else pending
        if self.norm2 is not None:
            n, n2 = self.norm.add_norm(resid, pending, act, second=self.norm2)
        else:
            n = n2 = self.norm.add_norm(resid, pending, act)
        a = self.mixer.forward(n, batch, cache, store)
        if self.ffn is None:
            return resid, a
        return resid, (a, self.ffn.forward(n2, batch))
