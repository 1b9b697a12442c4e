"""Mixture-of-experts feed-forward: a router picks `top` of `experts` small gated feed-forward layers per token.

    z = W_router h + b            (fp32 logits)
    picked = the `top` largest z; weights = softmax taken over those `top` values only
    y = sum_picked weight_e * down_e(act(gate_e h) * up_e h)  (+ shared(h), a gated feed-forward every token passes)

or, with score="softmax_all" (the routing of "DeepSeek-V3 Technical Report", DeepSeek-AI, with softmax scores):

    s = softmax(W_router h) over all experts;  the choice goes by s + correction (a per-expert offset that never enters the weights),
    restricted to the `keep` best of `groups` equal groups of neighbouring experts (a group's score: its largest corrected score);
    picked = the `top` best eligible;  weights = route_scale * s[picked], not renormalised;
    the shared expert's result is multiplied by sigmoid(W_sg h), one number per token (shared_gate=True).

or, with score="sigmoid": s = sigmoid(W_router h); picked = the `top` largest; weights = s[picked], not renormalised.

act="glu_clamp" is the capped gated unit  g = min(gate x, limit), u = clamp(up x, -limit, limit), y = g sigmoid(alpha g) (u + 1);
`weight_on_input` lets a choice's weight multiply the expert's INPUT instead of its result, y = sum_picked expert_e(weight_e h): the
first product is linear, so its rows are scaled by the weight before the caps apply, and the results are summed as they are.

The experts' matrices lie stacked, gate and up merged ([E, 2 ff, D] and [E, D, ff]), and run as two grouped products over
the (token, choice) pairs ordered by expert (ops.moe_align / ops.linear_grouped); routing, ordering and the tile list stay on
the device, so a step with experts needs no answer from the host and can be captured in a graph.  The result is the fp32
sum, meant to be added to an fp32 residual stream.
"""
from __future__ import annotations

import torch
from torch import nn

from .. import ops
from .activation import ActAndMul
from .linear import MergedLinear


class GatedMLP(nn.Module):
    """down(act(gate x) * up x) with gate and up in one product."""

    def __init__(self, width: int, ff: int, act: str = "silu"):
        super().__init__()
        self.gate_up = MergedLinear(width, [ff, ff], ["gate", "up"])
        self.act = ActAndMul(act)
        self.down = MergedLinear(ff, [width])

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.down(self.act(self.gate_up(x)))


class SparseMoE(nn.Module):
    def __init__(self, width: int, ff: int, experts: int, top: int, shared_ff: int | None = None, act: str = "silu", router_bias: bool = True,
                 score: str = "softmax_top", correction: bool = False, groups: int = 1, keep_groups: int = 1, route_scale: float = 1.0,
                 shared_gate: bool = False, limit: float | None = None, alpha: float = 1.702, weight_on_input: bool = False):
        super().__init__()
        assert 1 <= top <= experts and score in ("softmax_top", "softmax_all", "sigmoid")
        assert (act == "glu_clamp") == (limit is not None) and (not weight_on_input or act == "glu_clamp"), "limit belongs to act='glu_clamp', which alone takes the weight on the input"
        self.width, self.ff, self.experts, self.top, self.act, self.score = width, ff, experts, top, act, score
        self.limit, self.alpha, self.weight_on_input = limit, float(alpha), weight_on_input
        self.groups, self.keep_groups, self.route_scale = int(groups), int(keep_groups), float(route_scale)
        if score == "softmax_all":
            assert not router_bias and experts % self.groups == 0 and 1 <= self.keep_groups <= self.groups
            assert top <= self.keep_groups * (experts // self.groups), "fewer eligible experts than choices"
        else:
            assert not correction and self.groups == 1 and route_scale == 1.0, "these options belong to score='softmax_all'"
        self.router = MergedLinear(width, [experts], bias=router_bias)
        if correction:
            self.correction = nn.Parameter(torch.zeros(experts), requires_grad=False)
        else:
            self.register_parameter("correction", None)
        self.gate_up = nn.Parameter(torch.empty(experts, 2 * ff, width), requires_grad=False)
        self.down = nn.Parameter(torch.empty(experts, width, ff), requires_grad=False)
        self.gate_up.weight_loader = self._load_gate_up
        self.down.weight_loader = self._load_down
        self.gate_up.shard_ids = [(e, part) for e in range(experts) for part in ("gate", "up")]
        self.down.shard_ids = list(range(experts))
        assert not (shared_ff and act == "glu_clamp"), "the shared expert is a plain gated unit"
        self.shared = GatedMLP(width, shared_ff, act) if shared_ff else None
        self.shared_gate = MergedLinear(width, [1]) if (shared_gate and shared_ff) else None      # one logit per token

    def _load_gate_up(self, param: nn.Parameter, loaded_weight: torch.Tensor, shard_id):
        e, part = shard_id
        dst = param.data[e].narrow(0, 0 if part == "gate" else self.ff, self.ff)
        assert dst.shape == loaded_weight.shape, f"expert {e} {part}: {tuple(loaded_weight.shape)} does not fit {tuple(dst.shape)}"
        dst.copy_(loaded_weight)

    def _load_down(self, param: nn.Parameter, loaded_weight: torch.Tensor, shard_id):
        assert param.data[shard_id].shape == loaded_weight.shape
        param.data[shard_id].copy_(loaded_weight)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """x [T, width] in the activation type -> fp32 [T, width]."""
        gate = None
        if self.score == "softmax_all":
            ids, weights, gate = ops.moe_route_scored(x, self.router.weight.data, self.top, None if self.correction is None else self.correction.data,
                                                      self.groups, self.keep_groups, self.route_scale,
                                                      aux=None if self.shared_gate is None else self.shared_gate.weight.data)
        else:
            ids, weights = ops.moe_route_linear(x, self.router.weight.data, None if self.router.bias is None else self.router.bias.data, self.top,
                                                sigmoid_scores=self.score == "sigmoid")
            if self.shared_gate is not None:
                gate = self.shared_gate(x, out_f32=True)
        plan = ops.moe_align(ids, self.experts)
        first = ops.linear_grouped(x, self.gate_up.data, plan, gather=True)
        if self.act == "glu_clamp":
            hidden = ops.glu_clamp_pairs(first, plan, weights if self.weight_on_input else None, self.limit, self.alpha)
        else:
            hidden = ops.act_mul(first, self.act, True)
        y = ops.linear_grouped(hidden, self.down.data, plan, gather=False)
        return ops.moe_combine(y, plan, None if self.weight_on_input else weights, self.shared(x) if self.shared is not None else None, gate, top=self.top)
