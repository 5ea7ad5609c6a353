"""Gated feed-forward: down( silu(gate(x)) * up(x) ), no biases
(src/models/qwen3.hpp:232-263; src/backends/cpu/x64/kernels.cpp:242-247).
Gate and up run as one product with rows [gate | up].

``MoEMLP``: a mixture of such gated layers.  A router (float32) scores all experts, s = softmax(W_r x); the choice goes
by s plus a stored correction, among the experts of the best groups of neighbouring experts only; a token's result is
the sum of its chosen experts' results, weighted with the chosen s over their sum, times a constant."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import FeedForward


class GatedMLP(FeedForward):
    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu", fold_rows=None,
                 names=(".gate_proj.weight", ".up_proj.weight", ".down_proj.weight")):
        """``fold_rows``: most rows of a step whose products here run with the norms and the residual sum folded in
        (None: ``ops.default_fold_rows`` of this part's matrices).  ``names``: the tensors' names behind the prefix."""
        if activation != "silu":
            raise ValueError("GatedMLP: activation %r is not implemented" % activation)
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.fold_rows = fold_rows
        self.names = names
        self.w_gate_up = self.w_down = self.w_gate_up_tiled = self.w_down_tiled = None

    def weight_specs(self, prefix):
        H, I = self.hidden_size, self.intermediate_size
        gate, up, down = (prefix + n for n in self.names)
        return [WeightSpec(gate, (I, H)), WeightSpec(up, (I, H)), WeightSpec(down, (H, I))]

    def bind(self, prefix, weights):
        # (popped: the separate matrices are freed once they are fused, see PagedAttention.bind)
        gate, up, down = (prefix + n for n in self.names)
        g, u = weights.pop(gate), weights.pop(up)
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        self.w_gate_up = torch.cat([g, u], dim=0).contiguous()
        del g, u
        # tiles 0 .. I/16 - 1 of the tiled copy are gate rows, the rest up rows: what the fused SwiGLU kernel expects
        if self.intermediate_size % 16 == 0:
            self.w_gate_up, self.w_gate_up_tiled = ops.weight_forms(self.w_gate_up)
        self.w_down, self.w_down_tiled = ops.weight_forms(weights.pop(down))

    def capturable(self, batch):
        return True

    def can_fold(self, batch):
        return ops.fused_decode_ok(batch.T, batch.act_dtype, self.w_gate_up_tiled, self.w_down_tiled, max_rows=self.fold_rows)

    def forward(self, x, batch):
        if isinstance(x, ops.ScaledInput):
            return ops.linear(ops.decode_linear_swiglu(x, self.w_gate_up_tiled), self.w_down, tiled=self.w_down_tiled)
        return ops.linear_few(ops.linear_swiglu(x, self.w_gate_up, self.w_gate_up_tiled, few_rows=ops.DECODE_ROWS_PLAIN), self.w_down,
                              self.w_down_tiled)

    def forward_into(self, x, batch, resid, next_norm):
        weight, eps = next_norm.foldable(batch.act_dtype)
        return ops.decode_linear_residual(ops.decode_linear_swiglu(x, self.w_gate_up_tiled, for_product=True), self.w_down_tiled,
                                          resid, weight, eps, next_norm)


class DenseMLP(FeedForward):
    """down( act(up(x)) ), no gate and no biases.  ``activation`` "xielu": a piecewise activation with two learned
    numbers (p, q) in a tensor of its own: z > 0: softplus(p) z^2 + z/2; z <= 0: (1/2 + softplus(q)) (e^z - 1 - z) + z/2."""

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "xielu", names=("up", "down", "act")):
        if activation != "xielu":
            raise ValueError("DenseMLP: activation %r is not implemented" % activation)
        self.hidden_size, self.intermediate_size, self.names = hidden_size, intermediate_size, names
        self.w_up = self.w_up_tiled = self.w_down = self.w_down_tiled = self.act = None

    def weight_specs(self, prefix):
        H, I = self.hidden_size, self.intermediate_size
        up, down, act = (prefix + "." + n for n in self.names)
        return [WeightSpec(up, (I, H)), WeightSpec(down, (H, I)), WeightSpec(act, (2,), "bias")]

    def bind(self, prefix, weights):
        up, down, act = (prefix + "." + n for n in self.names)
        self.w_up, self.w_up_tiled = ops.weight_forms(weights.pop(up))
        self.w_down, self.w_down_tiled = ops.weight_forms(weights.pop(down))
        self.act = weights[act]

    def capturable(self, batch):
        return True

    def forward(self, x, batch):
        return ops.linear_few(ops.linear_xielu(x, self.w_up, self.act, tiled=self.w_up_tiled), self.w_down, self.w_down_tiled)


class MoEMLP(FeedForward):
    """``experts`` gated feed-forwards of inner size ``expert_size`` of which every token uses ``top``: those with the
    largest choice scores s + correction among the experts of the ``groups_kept`` best of ``groups`` equal groups of
    neighbours (a group's score is the largest choice score in it).  Weights: the chosen s over their sum (+ 1e-20),
    times ``scale``.  Tensors: ``router [experts, H]``, ``correction [experts]``, ``e<i>.gate``, ``e<i>.up``,
    ``e<i>.down``."""

    def __init__(self, hidden_size: int, expert_size: int, experts: int, top: int, groups: int = 1, groups_kept: int = 1,
                 scale: float = 1.0, names=("router", "correction", "e%d.gate", "e%d.up", "e%d.down"), score: str = "softmax",
                 renormalize: bool = True, correction: bool = True, weight_on: str = "output", activation: str = "silu",
                 limit: float = 0.0, router_bias: bool = False, shared: FeedForward = None, more_names=("router.b", "shared")):
        """``score``: "softmax" over all experts or "sigmoid" of each logit.  ``renormalize``: the chosen scores over their
        sum (else as they are), times ``scale``.  ``correction``: a stored vector is added to the scores for the choice.
        ``weight_on``: "output": out = sum w expert(x); "input": out = sum expert(w x).  ``activation``: "silu":
        silu(gate) * up; "clamped": g = min(gate, limit), u = clamp(up, -limit, limit), g sigmoid(1.702 g) (u + 1).
        ``router_bias``: the logits are W_r x + b (tensor ``router.b``); with softmax scores, renormalised, the weights are
        then the softmax over the chosen biased logits alone.  ``shared``: a feed-forward that every token uses (tensors
        under ``shared``), added to the experts' sum in the pass that forms it."""
        self.has_router_bias, self.shared, self.more_names = bool(router_bias), shared, more_names
        self.router_bias = None
        if score not in ("softmax", "sigmoid") or weight_on not in ("output", "input") or activation not in ("silu", "clamped"):
            raise ValueError("MoEMLP: score %r, weight_on %r or activation %r is not implemented" % (score, weight_on, activation))
        if activation == "clamped" and not limit > 0.0:
            raise ValueError("MoEMLP: the clamped activation needs a positive limit")
        self.score, self.renormalize, self.has_correction, self.weight_on = score, bool(renormalize), bool(correction), weight_on
        self.activation, self.limit = activation, float(limit)
        if experts <= 0 or groups <= 0 or experts % groups or not 0 < groups_kept <= groups or not 0 < top <= groups_kept * (experts // groups):
            raise ValueError("a choice of %d among %d of %d groups of %d experts cannot be made" % (top, groups_kept, groups, experts))
        self.hidden_size, self.expert_size, self.experts, self.top = hidden_size, expert_size, experts, top
        self.groups, self.groups_kept, self.scale, self.names = groups, groups_kept, float(scale), names
        self.w_router = self.correction = self.w_gate_up = self.w_down = None

    def weight_specs(self, prefix):
        H, F, E = self.hidden_size, self.expert_size, self.experts
        router, corr, gate, up, down = (prefix + "." + n for n in self.names)
        specs = [WeightSpec(router, (E, H))] + ([WeightSpec(corr, (E,), "bias")] if self.has_correction else [])
        for e in range(E):
            specs += [WeightSpec(gate % e, (F, H)), WeightSpec(up % e, (F, H)), WeightSpec(down % e, (H, F))]
        if self.has_router_bias:
            specs.append(WeightSpec(prefix + "." + self.more_names[0], (E,), "bias"))
        if self.shared is not None:
            specs += self.shared.weight_specs(prefix + "." + self.more_names[1])
        return specs

    def bind(self, prefix, weights):
        router, corr, gate, up, down = (prefix + "." + n for n in self.names)
        # the router's product keeps its float32 sums (bfloat16 operands multiply exactly in float32), and everything
        # behind it is float32: its scores decide, they are not activations
        self.w_router = weights.pop(router)
        self.correction = weights[corr].float().contiguous() if self.has_correction else None
        self.router_bias = weights[prefix + "." + self.more_names[0]].float().contiguous() if self.has_router_bias else None
        if self.shared is not None:
            self.shared.bind(prefix + "." + self.more_names[1], weights)
        E = self.experts
        mats = [weights.pop(n % e) for e in range(E) for n in (gate, up, down)]
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        # every expert's [gate rows | up rows] and its down matrix, the experts one after the other
        self.w_gate_up = torch.stack([torch.cat([mats[3 * e], mats[3 * e + 1]], dim=0) for e in range(E)]).contiguous()
        self.w_down = torch.stack([mats[3 * e + 2] for e in range(E)]).contiguous()

    def capturable(self, batch):
        return self.shared is None or self.shared.capturable(batch)

    def forward(self, x, batch):
        z = ops.linear(x, self.w_router, torch.float32)
        ids, weights = ops.moe_route(z, self.correction, self.top, self.groups, self.groups_kept, self.scale, score=self.score,
                                     renormalize=self.renormalize, logit_bias=self.router_bias)
        everyone = self.shared.forward(x, batch) if self.shared is not None else None
        return ops.moe_experts(x, ids, weights, self.w_gate_up, self.w_down, activation=self.activation, limit=self.limit,
                               weight_input=self.weight_on == "input", add=everyone)
