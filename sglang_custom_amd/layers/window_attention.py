"""WindowSinkAttention: the per-layer hand-off to the attention backend for softmax attention over a sliding window whose
denominator holds a sink term (RadixAttention's role, python/sglang/srt/layers/radix_attention.py:59-108, for a mechanism
the reference does not have):

    s_j = (q_i . k_j) * scale   for 0 <= i - j < window,      o_i = sum_j exp(s_j) v_j / (exp(sink_h) + sum_j exp(s_j))

No rotation: positions enter only through the window.  Query head h reads key / value head h // (heads / kv_heads); key and
value widths may differ.  sink is one fp32 logit per query head (a zero logit adds one to the denominator), or absent
(with_sink=False); window <= 0 means every earlier key.  Scores and weights are fp32 in every dtype."""
import torch
from torch import nn


class WindowSinkAttention(nn.Module):
    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, v_head_dim: int, scaling: float, window: int,
                 layer_id: int, device, with_sink: bool = True):
        super().__init__()
        assert num_heads % num_kv_heads == 0
        self.tp_q_head_num, self.tp_k_head_num, self.tp_v_head_num = num_heads, num_kv_heads, num_kv_heads
        self.qk_head_dim, self.v_head_dim = head_dim, v_head_dim
        self.scaling, self.window = float(scaling), int(window)
        self.layer_id = layer_id
        self.sink = nn.Parameter(torch.zeros(num_heads, dtype=torch.float32, device=device), requires_grad=False) if with_sink else None

    def forward(self, q: torch.Tensor, forward_batch, out: torch.Tensor) -> torch.Tensor:
        return forward_batch.attn_backend.forward_window(q, self, forward_batch, out)
