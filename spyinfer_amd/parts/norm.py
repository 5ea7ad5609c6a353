"""RMS norm.  y = x / sqrt(mean(x^2) + eps) * w, sums and scale in float32, eps inside the
root, the weight multiplies as it is (src/backends/cpu/x64/kernels.cpp:168-180;
src/backends/cuda/native/common.cuh:57-188)."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Norm


class RMSNorm(Norm):
    def __init__(self, size: int, eps: float, suffix: str = ".weight", offset: float = 0.0, groups: int = 1, scalar: bool = False):
        """``groups``: the vector is cut into that many equal consecutive parts, each over its own root mean square (the
        weight still spans the whole vector).  ``suffix``: what the weight's name has behind the part's prefix (some checkpoints name the vector by the
        prefix alone).  ``offset``: the stored vector is centred on zero and multiplies as ``offset + w`` (1.0 for norms
        whose weights are stored around zero); the sum is formed once, in float32, when the weights are bound.  ``scalar``:
        the stored weight is ONE number for all coordinates (a tensor without dimensions), spread over the vector when the
        weights are bound, so that the kernels see a weight vector as ever."""
        self.size = size
        self.eps = float(eps)
        self.suffix = suffix
        self.offset = float(offset)
        self.groups = int(groups)
        self.scalar = bool(scalar)
        if self.groups <= 0 or size % self.groups:
            raise ValueError("a norm in %d groups does not fit a vector of %d" % (self.groups, size))
        self.weight = None

    def weight_specs(self, prefix):
        # (the role says how random weights are drawn: around one, or around zero where the offset supplies the one)
        return [WeightSpec(prefix + self.suffix, () if self.scalar else (self.size,), "bias" if self.offset else "norm")]

    def bind(self, prefix, weights):
        self.weight = weights[prefix + self.suffix]
        if self.scalar:
            self.weight = self.weight.reshape(1).expand(self.size).contiguous()
        if self.offset:
            self.weight = (self.weight.float() + self.offset).contiguous()

    def capturable(self, batch):
        return True

    def add_norm(self, resid, delta, out_dtype, rows=None, second=None):
        """``delta``: None, one addend, a pair of addends (the results of two sublayers that read the same norm), or an
        ``ops.EntryAddends`` (any of these plus an earlier state of the stream and a vector for every row).  ``second``:
        another norm of this kind that reads the same sum: the result is the pair of both outputs, from one pass."""
        more = {}
        if isinstance(delta, ops.EntryAddends):
            more = dict(base=delta.base, vec=delta.vec)
            delta = None if isinstance(delta.pending, ops.ScaledInput) else delta.pending
            if isinstance(delta, ops.GatedAddend):
                delta = delta.resolve()
        if second is not None:
            if (second.size, second.eps, second.groups) != (self.size, self.eps, self.groups) or second.weight.dtype != self.weight.dtype:
                raise ValueError("two norms of one sum must have one size, eps, grouping and weight dtype")
            more["weight2"] = second.weight
        if more:
            if isinstance(delta, ops.GatedAddend):
                delta = delta.resolve()
            first, other = delta if isinstance(delta, (tuple, list)) else (delta, None)
            return ops.add_rms_norm(resid, first, self.weight, self.eps, out_dtype, rows, delta2=other, groups=self.groups, **more)
        if isinstance(delta, ops.GatedAddend):
            # a sublayer's result behind its gate: formed in this kernel's pass where the dtypes allow it
            if delta.bias.dtype != self.weight.dtype or not delta.gate.is_contiguous():
                delta = delta.resolve()
            else:
                return ops.add_rms_norm(resid, delta.y, self.weight, self.eps, out_dtype, rows, groups=self.groups,
                                        gate=(delta.gate, delta.bias, delta.mult))
        if isinstance(delta, (tuple, list)):
            first, second = delta
            return ops.add_rms_norm(resid, first, self.weight, self.eps, out_dtype, rows, delta2=second, groups=self.groups)
        return ops.add_rms_norm(resid, delta, self.weight, self.eps, out_dtype, rows, groups=self.groups)

    def add_normed(self, base, y, out=None, copy_dtype=None, mix=None):
        """out = base + norm(y) in float32 (the norm on a sublayer's output; ``out`` may be ``base``); returns (out, its
        copy in ``copy_dtype`` or None).  ``mix`` = (kept results [layers, T, H], n, weights [n]) with ``out`` the n-th
        kept result: the weighted sum of the n results is formed in the same pass and returned in place of ``out``."""
        if self.groups != 1:
            raise ValueError("a norm in groups on a sublayer's output is not implemented")
        if mix is not None and mix[2].dtype != self.weight.dtype:
            out, _ = ops.norm_residual(base, y, self.weight, self.eps, out, None)
            return ops.depth_mix(mix[0], mix[1], mix[2], copy_dtype)
        return ops.norm_residual(base, y, self.weight, self.eps, out, copy_dtype, mix)

    def foldable(self, out_dtype):
        if self.groups == 1 and not self.scalar and out_dtype == torch.bfloat16 and self.weight is not None and self.weight.dtype == torch.bfloat16:
            return self.weight, self.eps
        return None
