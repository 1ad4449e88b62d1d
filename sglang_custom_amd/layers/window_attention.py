"""WindowSinkAttention: the per-layer hand-off to the attention backend for softmax attention over a sliding window whose
denominator holds a sink term (RadixAttention's role, python/sglang/srt/layers/radix_attention.py:59-108, for a mechanism
the reference does not have):

    s_j = (q_i . k_j) * scale   for 0 <= i - j < window,      o_i = sum_j exp(s_j) v_j / (exp(sink_h) + sum_j exp(s_j))

No rotation: positions enter only through the window.  Query head h reads key / value head h // (heads / kv_heads); key and
value widths may differ.  sink is one fp32 logit per query head (a zero logit adds one to the denominator), or absent
(with_sink=False); window <= 0 means every earlier key.  Scores and weights are fp32 in every dtype.

pool > 0 (with a window): beside the window's tokens, token i sees one averaged key / value for every block b of `pool`
positions whose last position precedes its window (b pool + pool - 1 <= i - window), in the same softmax; a token behind
the window whose block still reaches into it is invisible until that block has passed.  The averages are rows of the cache pool's pooled
buffers, written by store_blocks() once a step's keys and values are in the cache, for every block length in store_pools
(the layer's own and those of the layers that read its cache under masks of their own).  kv_layer_id: the layer whose cached keys
and values (and averages) this layer reads when it has none of its own.  head_gate (logits [T, H], in forward): head h's
result times their sigmoid."""
from typing import Optional

import torch
from torch import nn


class WindowSinkAttention(nn.Module):
    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, v_head_dim: int, scaling: float, window: int,
                 layer_id: int, device, with_sink: bool = True, pool: int = 0, kv_layer_id: Optional[int] = None, store_pools=None):
        super().__init__()
        assert num_heads % num_kv_heads == 0
        self.tp_q_head_num, self.tp_k_head_num, self.tp_v_head_num = num_heads, num_kv_heads, num_kv_heads
        self.qk_head_dim, self.v_head_dim = head_dim, v_head_dim
        self.scaling, self.window = float(scaling), int(window)
        self.layer_id = layer_id
        self.pool = int(pool) if window > 0 else 0
        self.kv_layer_id = layer_id if kv_layer_id is None else int(kv_layer_id)
        self.store_pools = tuple(store_pools) if store_pools is not None else ((self.pool,) if self.pool > 0 else ())
        self.sink = nn.Parameter(torch.zeros(num_heads, dtype=torch.float32, device=device), requires_grad=False) if with_sink else None

    def forward(self, q: torch.Tensor, forward_batch, out: torch.Tensor, head_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
        return forward_batch.attn_backend.forward_window(q, self, forward_batch, out, head_gate=head_gate)

    def store_blocks(self, forward_batch) -> None:
        """After the step's keys and values went to the cache: the averages of the blocks that the step completes."""
        if self.store_pools:
            forward_batch.attn_backend.store_window_blocks(self, forward_batch)
