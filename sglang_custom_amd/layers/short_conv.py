"""ShortCausalConv: a causal convolution over time with one short filter per channel, for sequences that arrive in
pieces (no counterpart in the reference, whose models keep nothing but KV between steps):

    y_t = act( [u_t +] sum_{k < taps} w[:, taps - 1 - k] * u_{t - k} ),      u = 0 before the sequence's start

The last taps - 1 inputs of every sequence live in the sequence-state pool (SequenceStatePool.convs[key], fp32), are read
by a step's first tokens and replaced after the step; prefill portions, decode steps and mixed batches are the same call.
`second=True` holds a second filter over the same input (two results from one launch); `residual=True` adds the input to
each result (a convolution used as a correction of its input); `bias=True` adds a bias per channel to the (first) filter's
sum; act is "none" or "silu"."""
import torch
from torch import nn

from ..ops_backend import get_ops


class ShortCausalConv(nn.Module):
    def __init__(self, channels: int, taps: int, state_key, dtype, device, act: str = "none", residual: bool = False,
                 second: bool = False, bias: bool = False):
        super().__init__()
        assert taps >= 1 and act in ("none", "silu")
        self.channels, self.taps, self.state_key, self.act, self.residual = channels, int(taps), state_key, act, bool(residual)
        self.weight = nn.Parameter(torch.zeros(channels, taps, dtype=dtype, device=device), requires_grad=False)
        self.weight2 = nn.Parameter(torch.zeros(channels, taps, dtype=dtype, device=device), requires_grad=False) if second else None
        self.bias = nn.Parameter(torch.zeros(channels, dtype=dtype, device=device), requires_grad=False) if bias else None

    def forward(self, u: torch.Tensor, forward_batch):
        """u [T, channels] (row-strided) -> y, or (y, y2) with a second filter."""
        st = forward_batch.seq_state
        return get_ops().causal_conv(u, self.weight.data, st.pool.convs[self.state_key], st.req_to_state, st.req_pool_indices,
                                     forward_batch.positions, w2=self.weight2.data if self.weight2 is not None else None,
                                     residual=self.residual, act=self.act, **({"bias": self.bias.data} if self.bias is not None else {}),
                                     **st.segments())
