"""Plain, slow restatement of the Gatarax design for checking the product path: one function per mechanism, whole
sequences at once, no cache, no state hand-over, no batching, float64 by default.  Test infrastructure only; nothing
under sglang_custom_amd/ imports it and it imports nothing from there.

Notation: x [T, D] is the residual stream of ONE sequence at positions 0..T-1; weights come in a dict under their
checkpoint names (linear weights [out, in], applied as x @ W.T).

  stream      x_0 = E[token] * s_e;  per layer  h = N(x) (1 + w);  x <- x + mixer(h + C1(h)) + ff(h + C2(h))
  N           RMS norm, x / sqrt(mean(x^2) + eps)
  C           a causal convolution over time on every channel, zeros before the sequence
  mixer       "parallel": half the sum of two normed branches -- windowed softmax attention whose denominator holds an
              extra 1, and a gated delta rule with a decay per key channel; or "lightning": a linear recurrence with one
              fixed decay per head
  ff          squared-ReLU feed-forward, or a mixture of SiLU-gated experts chosen by softmax scores within the best groups
  output      logits = E (N(x) (1 + w_f)) * s_l
"""
import math
from typing import Dict, List, Optional

import torch


# ----------------------------------------------------------------------------------- small pieces
def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def relu_squared(z: torch.Tensor) -> torch.Tensor:
    return torch.clamp(z, min=0.0) ** 2


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """The weight is stored around zero."""
    return unit_rms(x, eps) * (1.0 + w)


def causal_conv(u: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """u [T, C], w [C, taps]; the LAST tap multiplies the current token, tap taps-1-k the token k steps back."""
    T, C = u.shape
    taps = w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for k in range(taps):
            if t - k >= 0:
                y[t] += w[:, taps - 1 - k] * u[t - k]
    return y


# ----------------------------------------------------------------------------------- mixers
def window_sink_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: int) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv].  Token i sees j with 0 <= i - j < window; the weights are
    exp(s_j) / (1 + sum exp(s_j)): a key of score 0 without a value sits in every row."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            lo = max(0, i - window + 1)
            s = (k[lo:i + 1, g] @ q[i, h]) * scale
            m = max(float(s.max()), 0.0)
            e = torch.exp(s - m)
            out[i, h] = (e[:, None] * v[lo:i + 1, g]).sum(0) / (math.exp(-m) + e.sum())
    return out


def gated_delta_rule(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, beta: torch.Tensor, decay: torch.Tensor) -> torch.Tensor:
    """q, k [T, G, d] (already unit vectors, q scaled), v [T, H, dv], beta [T, H], decay [T, H, d] -> [T, H, dv].
    Per head, with S [d, dv] zero at the start:  S <- diag(decay_t) S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;
    o_t = S^T q_t."""
    T, H, dv = v.shape
    G, d = k.shape[1], k.shape[2]
    out = torch.zeros(T, H, dv, dtype=v.dtype)
    for h in range(H):
        g = h // (H // G)
        S = torch.zeros(d, dv, dtype=v.dtype)
        for t in range(T):
            S = decay[t, h][:, None] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, h] = S.T @ q[t, g]
    return out


def decayed_sum(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor) -> torch.Tensor:
    """o_t = sum_{j <= t} decay_h^(t - j) (q_t . k_j) v_j: the closed form of S_t = decay S_{t-1} + k_t v_t^T, o_t = S_t^T q_t."""
    T, H, _ = q.shape
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    steps = torch.arange(T, dtype=q.dtype)
    for h in range(H):
        for t in range(T):
            wgt = decay[h] ** (t - steps[: t + 1]) * (k[: t + 1, h] @ q[t, h])
            out[t, h] = (wgt[:, None] * v[: t + 1, h]).sum(0)
    return out


def unit_vectors(x: torch.Tensor) -> torch.Tensor:
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def left_branch(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mx: dict) -> torch.Tensor:
    T = h.shape[0]
    H, G, d, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = causal_conv(h @ w[p + "q"].T + w[p + "q.b"], w[p + "q.conv"]).reshape(T, H, d)
    k = causal_conv(h @ w[p + "k"].T + w[p + "k.b"], w[p + "k.conv"]).reshape(T, G, d)
    v = causal_conv(h @ w[p + "v"].T + w[p + "v.b"], w[p + "v.conv"]).reshape(T, G, dv)
    o = window_sink_attention(q, k, v, mx["scale"], mx["mask"]["size"])
    return o.reshape(T, H * dv) @ w[p + "o"].T + w[p + "o.b"]


def right_branch(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mx: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, d, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = silu(causal_conv(h @ w[p + "q"].T, w[p + "q.conv"])).reshape(T, G, d)
    k = silu(causal_conv(h @ w[p + "k"].T, w[p + "k.conv"])).reshape(T, G, d)
    v = silu(causal_conv(h @ w[p + "v"].T, w[p + "v.conv"])).reshape(T, H, dv)
    q = unit_vectors(q) * d ** -0.5
    k = unit_vectors(k)
    beta = torch.sigmoid(h @ w[p + "b"].T)
    z = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]
    rate = torch.exp(w[p + "A_log"])[None, :, None] * torch.nn.functional.softplus(z).reshape(T, H, d)
    o = gated_delta_rule(q, k, v, beta, torch.exp(-rate))
    gate = torch.sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T).reshape(T, H, dv)
    o = unit_rms(o, eps) * w[p + "norm"] * gate
    return o.reshape(T, H * dv) @ w[p + "o"].T


def parallel_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mx: dict, eps: float) -> torch.Tensor:
    a = left_branch(h, w, p + "left.", mx["left"])
    b = right_branch(h, w, p + "right.", mx["right"], eps)
    return 0.5 * (unit_rms(a, eps) * w[p + "left.out"] + unit_rms(b, eps) * w[p + "right.out"])


def lightning_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mx: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, d, dv = mx["heads"], mx["dim"], mx["vdim"]
    q = silu(h @ w[p + "q"].T).reshape(T, H, d)
    k = silu(h @ w[p + "k"].T).reshape(T, H, d)
    v = silu(h @ w[p + "v"].T).reshape(T, H, dv)
    o = decayed_sum(q, k, v, torch.tensor(mx["decay"], dtype=h.dtype)).reshape(T, H * dv)
    o = unit_rms(o, eps) * w[p + "norm"] * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


# ----------------------------------------------------------------------------------- feed-forward
def dense_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    return relu_squared(h @ w[p + "up"].T) @ w[p + "down"].T


def route(scores: torch.Tensor, top: int, n_groups: int, keep: int):
    """scores [T, E] -> (ids [T, top], weights [T, top]).  A group of neighbouring experts counts by its best member; only
    the `keep` best groups stay eligible; the weights are the scores themselves."""
    T, E = scores.shape
    per = E // n_groups
    best = scores.reshape(T, n_groups, per).max(-1).values
    kept = torch.topk(best, keep, dim=-1).indices
    allowed = torch.zeros(T, n_groups, dtype=torch.bool)
    allowed.scatter_(1, kept, True)
    masked = torch.where(allowed[:, :, None].expand(T, n_groups, per).reshape(T, E), scores, torch.full_like(scores, -1.0))
    ids = torch.topk(masked, top, dim=-1).indices
    return ids, torch.gather(scores, 1, ids)


def moe_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mlp: dict, router_input: Optional[torch.Tensor] = None) -> torch.Tensor:
    r = mlp["router"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    hr = h if router_input is None else router_input
    scores = torch.softmax(hr @ w[p + "router"].to(hr.dtype).T, dim=-1)
    ids, wts = route(scores, r["top"], groups["count"], groups["keep"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(r["top"]):
            e = int(ids[t, j])
            a = silu(h[t] @ w[f"{p}e{e}.gate"].T) * (h[t] @ w[f"{p}e{e}.up"].T)
            out[t] += wts[t, j].to(h.dtype) * (a @ w[f"{p}e{e}.down"].T)
    return out


# ----------------------------------------------------------------------------------- the model
def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64, streams: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence.  `streams` (a list) receives the residual stream after every layer."""
    w = {n: (t.to(dtype) if t.is_floating_point() else t) for n, t in weights.items()}
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = offset_rms_norm(x, w[p + "norm1"], eps)
        hm = h + causal_conv(h, w[p + "canon1"])
        if spec["type"] == "parallel":
            y = parallel_mixer(hm, w, p + "mix.", spec["mixer"], eps)
        elif spec["type"] == "lightning":
            y = lightning_mixer(hm, w, p + "mix.", spec["mixer"], eps)
        else:
            raise ValueError(spec["type"])
        mlp = spec.get("mlp")
        if mlp is not None:
            hf = h + causal_conv(h, w[p + "canon2"])
            y = y + (dense_ff(hf, w, p + "mlp.") if mlp["kind"] == "dense" else moe_ff(hf, w, p + "mlp.", mlp))
        x = x + y
        if streams is not None:
            streams.append(x.clone())
    return (offset_rms_norm(x, w["final.norm"], eps) @ w["embed"].T) * cfg.get("logit_scale", 1.0)


def greedy(cfg: dict, weights: Dict[str, torch.Tensor], prompt: List[int], n: int) -> List[int]:
    """n tokens by argmax, each from a fresh whole-sequence forward."""
    toks, out = list(prompt), []
    for _ in range(n):
        nxt = int(torch.argmax(forward(cfg, weights, toks)[-1]))
        out.append(nxt)
        toks.append(nxt)
    return out
