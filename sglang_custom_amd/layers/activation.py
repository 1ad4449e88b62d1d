"""SiluAndMul (python/sglang/srt/layers/activation.py:55-65): x [.., 2d] -> [.., d]; Activation: a plain elementwise
function of a projection's output ("silu", or "relu2", the square of relu)."""
import torch

from ..custom_op import CustomOp
from ..ops_backend import get_ops


class SiluAndMul(CustomOp):
    def forward_hip(self, x: torch.Tensor) -> torch.Tensor:
        if not x.is_contiguous():
            x = x.contiguous()
        return get_ops().silu_and_mul(x)


class GeluTanhAndMul(CustomOp):
    """gelu_tanh(gate) * up with gelu_tanh(z) = 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))); gate and up are
    column blocks of one projection's output."""

    def forward_hip(self, gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        return get_ops().gelu_tanh_and_mul(gate, up)


class Activation(CustomOp):
    def __init__(self, kind: str):
        super().__init__()
        assert kind in ("silu", "relu2")
        self.kind = kind

    def forward_hip(self, x: torch.Tensor) -> torch.Tensor:
        """x [T, d] (row-strided: a column block of a wider projection will do) -> contiguous [T, d]."""
        return get_ops().activation(x, self.kind)
