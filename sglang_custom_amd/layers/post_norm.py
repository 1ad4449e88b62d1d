"""Norms of a model that normalises AFTER the residual sum, on an fp32 residual stream (no counterpart in the
reference, whose models norm before their sublayers and keep the residual in the activation dtype):

  GroupRMSNorm        x <- N(c x + branch) * w in place, N = RMS norm over `groups` equal consecutive parts of the row,
                      each divided by its own sqrt(mean(part^2) + eps).  The branch is a [T, D] tensor or a weighted sum
                      of rows of a larger tensor (the chosen experts' outputs of a mixture).  One launch, which also
                      writes the activation-dtype copy of the new x that the next projections read.
  NormedResidualAdd   x <- x + mult * ls * y / sqrt(mean(y^2) + eps) * (offset + w) in place, same second output: a norm on a
                      sublayer's OUTPUT; offset 1 for a weight stored around zero, ls an optional per-channel layer scale.

groups, eps and c are constructor arguments; all arithmetic is fp32 whatever the activation dtype."""
from typing import Optional

import torch
from torch import nn

from ..ops_backend import get_ops


class GroupRMSNorm(nn.Module):
    def __init__(self, hidden: int, groups: int, eps: float, dtype, device, residual_scale: float = 1.0):
        super().__init__()
        assert groups >= 1 and hidden % groups == 0
        self.groups, self.eps, self.residual_scale = int(groups), float(eps), float(residual_scale)
        self.weight = nn.Parameter(torch.ones(hidden, dtype=dtype, device=device), requires_grad=False)

    def forward(self, x: torch.Tensor, branch: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None,
                coef: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x fp32 [T, D], updated in place; returns its copy in the weight's dtype.  rows int32 [T, n] / coef fp32 [T, n]:
        the branch of token t is sum_j coef[t, j] * branch[rows[t, j]]."""
        return get_ops().scaled_add_group_rmsnorm(x, branch, self.residual_scale, self.weight.data, self.groups, self.eps,
                                                  rows=rows, coef=coef, inplace=True)

    def normed(self, x: torch.Tensor) -> torch.Tensor:
        """N(x) * w in the weight's dtype; x is left as it is (a model's last norm)."""
        return get_ops().scaled_add_group_rmsnorm(x, None, 1.0, self.weight.data, self.groups, self.eps, inplace=False)


class NormedResidualAdd(nn.Module):
    def __init__(self, hidden: int, eps: float, dtype, device, offset: float = 0.0, mult: float = 1.0, layer_scale: bool = False):
        super().__init__()
        self.eps, self.offset, self.mult = float(eps), float(offset), float(mult)
        self.weight = nn.Parameter((torch.zeros if offset else torch.ones)(hidden, dtype=dtype, device=device), requires_grad=False)
        self.layer_scale = nn.Parameter(torch.ones(hidden, dtype=dtype, device=device), requires_grad=False) if layer_scale else None

    def forward(self, x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
        if self.offset == 0.0 and self.mult == 1.0 and self.layer_scale is None:
            return get_ops().rmsnorm_residual_add(x, y, self.weight.data, self.eps)
        return get_ops().rmsnorm_residual_add(x, y, self.weight.data, self.eps, offset=self.offset, mult=self.mult,
                                              layer_scale=self.layer_scale.data if self.layer_scale is not None else None)
