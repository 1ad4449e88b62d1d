"""Mixture of experts with a grouped top-k router (the role of the reference's python/sglang/srt/layers/moe/: topk.py
grouped_topk / biased_grouped_topk and fused_moe_triton/layer.py FusedMoE, re-done for this package's kernels).

  GroupedTopKRouter   scores s = sigmoid(x W_r^T) in fp32.  Selection runs on s + correction; experts form `n_groups`
                      equal groups of neighbours, a group scores the sum of its two largest selection scores, only
                      experts of the `keep_groups` best groups can be chosen (the others count as -inf), the `top`
                      largest are taken.  Weights: the chosen experts' s (without the correction) over their sum
                      (+ 1e-20), times `scale`.  Variants by constructor argument: scores = softmax over all experts
                      (score_fn="softmax"), no correction (with_correction=False), a group scoring its best member alone
                      (group_best=1), weights left as the chosen scores times `scale` (renorm=False).
  GroupedExperts      expert e: down_e(act(up_e(h))), act = erf-GELU.  Tokens are sorted by expert on the device into
                      blocks of `block` rows that belong to one expert each (ops.moe_align); two grouped GEMMs run over
                      the blocks (the first gathers its rows and applies the activation in its epilogue); the weighted
                      sum over a token's experts is left to the norm kernel that consumes it
                      (GroupRMSNorm.forward(rows=, coef=)), in a fixed order.  Nothing is read back to the host.
                      activation="silu_gated": down_e(silu(gate_e(h)) * up_e(h)), gate and up stacked in one weight."""
from typing import Tuple

import torch
from torch import nn

from ..ops_backend import get_ops


class GroupedTopKRouter(nn.Module):
    def __init__(self, hidden: int, num_experts: int, top: int, n_groups: int, keep_groups: int, scale: float, device,
                 score_fn: str = "sigmoid", group_best: int = 2, renorm: bool = True, with_correction: bool = True):
        super().__init__()
        assert num_experts % n_groups == 0 and 1 <= keep_groups <= n_groups and 1 <= top <= num_experts // n_groups * keep_groups
        assert score_fn in ("sigmoid", "softmax") and group_best in (1, 2)
        self.num_experts, self.top, self.n_groups, self.keep_groups, self.scale = num_experts, top, n_groups, keep_groups, float(scale)
        self.score_fn, self.group_best, self.renorm = score_fn, int(group_best), bool(renorm)
        # fp32 whatever the model dtype: the router's logits are computed in fp32 from the fp32 residual stream
        self.weight = nn.Parameter(torch.zeros(num_experts, hidden, dtype=torch.float32, device=device), requires_grad=False)
        self.correction = (nn.Parameter(torch.zeros(num_experts, dtype=torch.float32, device=device), requires_grad=False)
                           if with_correction else None)

    def forward(self, x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        """x fp32 [T, D] -> (expert ids int32 [T, top], weights fp32 [T, top])."""
        ops = get_ops()
        logits = ops.moe_router_logits(x, self.weight.data)
        if self.score_fn == "sigmoid" and self.group_best == 2 and self.renorm and self.correction is not None:
            return ops.moe_route_grouped(logits, self.correction.data, self.top, self.n_groups, self.keep_groups, self.scale)
        return ops.moe_route_scores(logits, self.correction.data if self.correction is not None else None, self.top, self.n_groups,
                                    self.keep_groups, self.scale, score_fn=self.score_fn, group_best=self.group_best,
                                    renorm=self.renorm)


class GroupedExperts(nn.Module):
    def __init__(self, hidden: int, ff: int, num_experts: int, dtype, device, activation: str = "gelu_erf"):
        super().__init__()
        assert activation in ("gelu_erf", "silu_gated")
        self.num_experts, self.hidden, self.ff, self.activation = num_experts, hidden, ff, activation
        # silu_gated: rows [gate (ff) | up (ff)] of every expert in one weight, as the dense models stack gate_up
        up_rows = 2 * ff if activation == "silu_gated" else ff
        self.w_up = nn.Parameter(torch.zeros(num_experts, up_rows, hidden, dtype=dtype, device=device), requires_grad=False)
        self.w_down = nn.Parameter(torch.zeros(num_experts, hidden, ff, dtype=dtype, device=device), requires_grad=False)

    def forward(self, h: torch.Tensor, expert_ids: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        """h [T, D], expert_ids int32 [T, top] -> (y [P, D], rows int32 [T, top]): y[rows[t, j]] is the output of token
        t's j-th expert; P >= T * top counts the padding of the experts' blocks."""
        ops = get_ops()
        sixteen = h.dtype != torch.float32
        plan = ops.moe_align(expert_ids, self.num_experts, wide_ok=sixteen and self.hidden % 8 == 0 and self.ff % 8 == 0,
                             tiled_ok=sixteen and h.shape[0] > 64 and h.stride(0) % 8 == 0
                             and ops.linear_tiled_supported(256, self.w_up.shape[1], self.hidden, h.dtype)
                             and ops.linear_tiled_supported(256, self.hidden, self.ff, h.dtype))
        if self.activation == "silu_gated":
            a = ops.silu_and_mul(ops.moe_grouped_linear(h, self.w_up.data, plan, gather=True, gelu=False))
        else:
            a = ops.moe_grouped_linear(h, self.w_up.data, plan, gather=True, gelu=True)
        y = ops.moe_grouped_linear(a, self.w_down.data, plan, gather=False, gelu=False)
        return y, plan.rows
