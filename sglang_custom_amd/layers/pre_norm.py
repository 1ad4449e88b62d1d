"""Norm and residual sum of a model that norms BEFORE its sublayers on an fp32 residual stream and runs several branches
off one norm (no counterpart in the reference, whose models keep the residual in the activation dtype):

  OffsetRMSNorm       h = x / sqrt(mean(x^2) + eps) * (offset + w): a weight stored around zero (offset 1) or plain
                      (offset 0); fp32 in, activation dtype out.
  BranchResidualAdd   x += s * (A + B) + F in place: A and B are branch outputs, each optionally divided by its own root
                      mean square and multiplied by a weight (a normed branch), F a feed-forward's output given as rows
                      or as a weighted sum of picked rows (a token's experts).  One launch; all arithmetic fp32."""
from typing import Optional

import torch
from torch import nn

from ..ops_backend import get_ops


class OffsetRMSNorm(nn.Module):
    def __init__(self, hidden: int, eps: float, dtype, device, offset: float = 1.0):
        super().__init__()
        self.eps, self.offset = float(eps), float(offset)
        self.weight = nn.Parameter(torch.zeros(hidden, dtype=dtype, device=device), requires_grad=False)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return get_ops().offset_rmsnorm(x, self.weight.data, self.eps, self.offset)


class BranchResidualAdd(nn.Module):
    def __init__(self, hidden: int, eps: float, dtype, device, normed_branches: int = 0, scale: float = 1.0):
        super().__init__()
        assert normed_branches in (0, 1, 2)
        self.eps, self.scale = float(eps), float(scale)
        self.weight_a = nn.Parameter(torch.ones(hidden, dtype=dtype, device=device), requires_grad=False) if normed_branches >= 1 else None
        self.weight_b = nn.Parameter(torch.ones(hidden, dtype=dtype, device=device), requires_grad=False) if normed_branches >= 2 else None

    def forward(self, x: torch.Tensor, a: torch.Tensor, b: Optional[torch.Tensor] = None, f: Optional[torch.Tensor] = None,
                rows: Optional[torch.Tensor] = None, coef: Optional[torch.Tensor] = None) -> torch.Tensor:
        return get_ops().branch_residual_add(x, a, self.weight_a.data if self.weight_a is not None else None, b,
                                             self.weight_b.data if self.weight_b is not None else None, self.scale, f=f, rows=rows,
                                             coef=coef, eps=self.eps)
