"""LinearRecurrence: the per-layer hand-off to the recurrence kernel for mixers that keep one matrix per head and
sequence instead of keys and values per token (no counterpart in the reference, whose models keep nothing but KV):

    S_t = diag(a_t) S_{t-1} + k_t v_t^T          S [key width, value width], fp32, zero before position 0
    o_t = S_t^T (q_t * q_scale)

with the decay a_t either per key channel and token, a_t = sigmoid(z_t + b)^(1 / tau) from gate logits z (gated linear
attention), or one fixed number per head (retention).  The matrices live in the sequence-state pool
(SequenceStatePool.matrices[layer]); a step reads a sequence's matrix (or starts from zero at position 0), runs the
step's tokens of that sequence through it and writes it back, so prefill portions, decode steps and mixed batches are
the same launch.  Decays, their logarithms and the state are fp32 in every dtype.

GatedDeltaRule: the same hand-off for the delta rule with a decay per key channel,

    S <- diag(a_t) S;   u_t = beta_t (v_t - S^T k_t);   S <- S + k_t u_t^T;   o_t = S^T (q_t * q_scale)

with a_t = exp(-exp(rate_log_h) * softplus(z_t + rate_bias)) from fp32 logits z and beta_t = sigmoid of one logit per head;
q and k may have fewer heads than v (grouped).

StateSpaceRecurrence: the same hand-off for the state-space form with one scalar decay per head and token from a step
size, dt_t = softplus(z_t + dt_bias), a_t = exp(-exp(rate_log_h) dt_t):

    S_t = a_t S_{t-1} + dt_t B_t x_t^T;   y_t = S_t^T C_t + skip_h x_t

B and C (the keys and the queries) may be shared by groups of heads.

GatedGroupNorm: y * silu(gate), THEN an RMS norm over `groups` equal parts of the row, times a weight.

HeadNormGate: the recurrence's fp32 output per head divided by its root mean square (times a weight shared by the heads,
if there is one), times silu(gate) or sigmoid(gate), in the activation dtype for the output projection."""
from typing import Optional

import torch
from torch import nn

from ..ops_backend import get_ops
from .rotary_embedding import pair_inv_freq


class LinearRecurrence(nn.Module):
    def __init__(self, num_heads: int, key_dim: int, value_dim: int, layer_id: int, device, q_scale: float = 1.0,
                 head_decay=None, tau: float = 1.0):
        super().__init__()
        self.num_heads, self.key_dim, self.value_dim, self.layer_id = num_heads, key_dim, value_dim, layer_id
        self.q_scale, self.tau = float(q_scale), float(tau)
        assert head_decay is None or len(head_decay) == num_heads
        self.register_buffer("head_decay", None if head_decay is None else
                             torch.tensor(list(head_decay), dtype=torch.float32, device=device), persistent=False)

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, forward_batch, gate_logits=None, gate_bias=None):
        """q, k [T, H, dk], v [T, H, dv] (any token stride) -> fp32 [T, H, dv]."""
        st = forward_batch.seq_state
        out = torch.empty((q.shape[0], self.num_heads, self.value_dim), dtype=torch.float32, device=q.device)
        get_ops().linear_recurrence(q, k, v, out, st.pool.matrices[self.layer_id], st.req_to_state, st.req_pool_indices,
                                    forward_batch.positions, self.q_scale, gate_logits=gate_logits, gate_bias=gate_bias,
                                    tau=self.tau, head_decay=self.head_decay, **st.segments())
        return out


class StateSpaceRecurrence(nn.Module):
    def __init__(self, num_heads: int, groups: int, state_dim: int, value_dim: int, layer_id: int, device):
        super().__init__()
        assert num_heads % groups == 0
        self.num_heads, self.groups, self.state_dim, self.value_dim, self.layer_id = num_heads, groups, state_dim, value_dim, layer_id
        # fp32 whatever the model dtype: they enter the decay and the state
        self.rate_log = nn.Parameter(torch.zeros(num_heads, dtype=torch.float32, device=device), requires_grad=False)
        self.dt_bias = nn.Parameter(torch.zeros(num_heads, dtype=torch.float32, device=device), requires_grad=False)
        self.skip = nn.Parameter(torch.zeros(num_heads, dtype=torch.float32, device=device), requires_grad=False)

    def forward(self, c: torch.Tensor, b: torch.Tensor, x: torch.Tensor, dt_logits: torch.Tensor, forward_batch):
        """c, b [T, G, N] (read-out and write vectors), x [T, H, dv], dt_logits fp32 [T, H] -> fp32 [T, H, dv]."""
        st = forward_batch.seq_state
        out = torch.empty((x.shape[0], self.num_heads, self.value_dim), dtype=torch.float32, device=x.device)
        get_ops().linear_recurrence(c, b, x, out, st.pool.matrices[self.layer_id], st.req_to_state, st.req_pool_indices,
                                    forward_batch.positions, 1.0, dt_logits=dt_logits, dt_bias=self.dt_bias.data,
                                    rate_log=self.rate_log.data, skip=self.skip.data, **st.segments())
        return out


class GatedGroupNorm(nn.Module):
    def __init__(self, hidden: int, groups: int, eps: float, dtype, device):
        super().__init__()
        assert groups >= 1 and hidden % groups == 0
        self.groups, self.eps = int(groups), float(eps)
        self.weight = nn.Parameter(torch.ones(hidden, dtype=dtype, device=device), requires_grad=False)

    def forward(self, y: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
        """y fp32 [T, D], gate [T, D] logits (row-strided) -> [T, D] in the weight's dtype."""
        return get_ops().gated_group_rmsnorm(y, gate, self.weight.data, self.groups, self.eps)


class GatedDeltaRule(nn.Module):
    def __init__(self, num_heads: int, qk_heads: int, key_dim: int, value_dim: int, layer_id: int, device, q_scale: float = 1.0,
                 decay_per_head: bool = False):
        super().__init__()
        assert num_heads % qk_heads == 0
        self.num_heads, self.qk_heads, self.key_dim, self.value_dim, self.layer_id = num_heads, qk_heads, key_dim, value_dim, layer_id
        self.q_scale = float(q_scale)
        # fp32 whatever the model dtype: they enter the decay
        self.rate_log = nn.Parameter(torch.zeros(num_heads, dtype=torch.float32, device=device), requires_grad=False)
        # one decay per key channel, or (decay_per_head) one per head: the logits are then [T, H]
        self.rate_bias = nn.Parameter(torch.zeros(num_heads if decay_per_head else num_heads * key_dim, dtype=torch.float32,
                                                  device=device), requires_grad=False)

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, beta_logits: torch.Tensor, gate_logits: torch.Tensor,
                forward_batch):
        """q, k [T, G, dk], v [T, H, dv], beta_logits [T, H], gate_logits fp32 [T, H * dk] (or [T, H]) -> fp32 [T, H, dv]."""
        st = forward_batch.seq_state
        out = torch.empty((q.shape[0], self.num_heads, self.value_dim), dtype=torch.float32, device=q.device)
        get_ops().gated_delta_rule(q, k, v, beta_logits, gate_logits, self.rate_bias.data, self.rate_log.data, out,
                                   st.pool.matrices[self.layer_id], st.req_to_state, st.req_pool_indices, forward_batch.positions,
                                   self.q_scale, **st.segments())
        return out


class HeadNormGate(nn.Module):
    def __init__(self, value_dim: int, eps: float, dtype, device, with_weight: bool, gate_act: str = "silu"):
        super().__init__()
        assert gate_act in ("silu", "sigmoid")
        self.gate_act = gate_act
        self.eps = float(eps)
        self.out_dtype = dtype
        self.weight = (nn.Parameter(torch.ones(value_dim, dtype=dtype, device=device), requires_grad=False)
                       if with_weight else None)

    def forward(self, o: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
        """o fp32 [T, H, dv], gate [T, H * dv] logits (row-strided) -> [T, H * dv]."""
        w = self.weight.data if self.weight is not None else None
        if self.gate_act == "silu":
            return get_ops().head_rmsnorm_gate(o, w, gate, self.eps, self.out_dtype)
        return get_ops().head_rmsnorm_gate_act(o, w, gate, self.eps, self.out_dtype, self.gate_act)


class QKVHeadNormRope(nn.Module):
    """The head norms of an attention layer whose queries and keys are RMS-normed per head (weights shared by the heads, one for
    q, one for k) and rotated alike, and whose values are divided by their root mean square: one launch that returns the
    queries and writes keys and values into their cache rows.  Rotation as HeadNormRope's (frequencies base^(-2 i / rot_dims)
    or a given table, cos and sin times rot_mag)."""

    def __init__(self, head_dim: int, v_head_dim: int, rot_dims: int, rot_base: float, interleaved: bool, eps: float, dtype, device,
                 inv_freq: Optional[torch.Tensor] = None, rot_mag: float = 1.0):
        super().__init__()
        assert 0 <= rot_dims <= head_dim and rot_dims % 2 == 0
        self.head_dim, self.v_head_dim, self.rot_dims, self.interleaved = head_dim, v_head_dim, rot_dims, interleaved
        self.eps, self.rot_mag = float(eps), float(rot_mag)
        self.q_weight = nn.Parameter(torch.ones(head_dim, dtype=dtype, device=device), requires_grad=False)
        self.k_weight = nn.Parameter(torch.ones(head_dim, dtype=dtype, device=device), requires_grad=False)
        self.register_buffer("inv_freq", (pair_inv_freq(rot_base, rot_dims) if inv_freq is None else inv_freq.to(torch.float32)).to(device),
                             persistent=False)

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, positions: torch.Tensor, k_cache: torch.Tensor,
                v_cache: torch.Tensor, loc: torch.Tensor) -> torch.Tensor:
        """q [T, H, d], k [T, G, d], v [T, G, dv] (any token stride) -> normed and rotated q [T, H, d]."""
        return get_ops().qkv_norm_rope_write(q, k, v, self.q_weight.data, self.k_weight.data, self.eps, positions, self.inv_freq,
                                             self.rot_dims, self.interleaved, self.rot_mag, k_cache, v_cache, loc)


class HeadNormRope(nn.Module):
    """Per token and head: an optional RMS norm over the head's features with a weight shared by the heads, then a
    rotation of the first rot_dims features by position * base^(-2 i / rot_dims) (feature 2 i with 2 i + 1 when
    `interleaved`, else i with i + rot_dims / 2; angles in fp32 from the position, no table), then a scale.  One
    launch; the result goes to a new tensor or straight into cache rows."""

    def __init__(self, head_dim: int, rot_dims: int, rot_base: float, interleaved: bool, eps: float, dtype, device,
                 with_norm: bool, scale: float = 1.0, inv_freq: Optional[torch.Tensor] = None, rot_mag: float = 1.0):
        """inv_freq: the rotation's frequencies when they are not base^(-2 i / rot_dims) (scaled for longer sequences), with
        rot_mag the factor on cos and sin that comes with them."""
        super().__init__()
        assert 0 <= rot_dims <= head_dim and rot_dims % 2 == 0
        self.head_dim, self.rot_dims, self.interleaved, self.eps, self.scale = head_dim, rot_dims, interleaved, float(eps), float(scale)
        self.weight = nn.Parameter(torch.ones(head_dim, dtype=dtype, device=device), requires_grad=False) if with_norm else None
        self.rot_mag = float(rot_mag)
        self.register_buffer("inv_freq", (pair_inv_freq(rot_base, rot_dims) if inv_freq is None else inv_freq.to(torch.float32)).to(device),
                             persistent=False)

    def forward(self, src: torch.Tensor, positions: torch.Tensor, out_dtype, cache: Optional[torch.Tensor] = None,
                loc: Optional[torch.Tensor] = None) -> torch.Tensor:
        """src [T, H, d] (any token stride) -> [T, H, d] of out_dtype, or written to cache[loc[t]] when a cache is given."""
        return get_ops().head_norm_rope(src, self.weight.data if self.weight is not None else None, self.eps, positions,
                                        self.inv_freq, self.rot_dims, self.interleaved, self.scale, out_dtype, cache=cache, loc=loc,
                                        **({"rot_mag": self.rot_mag} if self.rot_mag != 1.0 else {}))
