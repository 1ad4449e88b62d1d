"""Plain, slow restatement of the Fudonex design for checking the product path: one function per mechanism, whole
sequences at once, no cache, no state hand-over, no batching, float64 by default.  Test infrastructure only; nothing
under sglang_custom_amd/ imports it and it imports nothing from there.

Notation: x [T, D] is the residual stream of ONE sequence at positions 0..T-1; weights come in a dict under their
checkpoint names (linear weights [out, in], applied as x @ W.T).

  stream      x_0 = E[token] * s_e;  per layer  x <- x + m * l1 * N(mixer(x)) (1 + w1);  x <- x + m * l2 * N(ff(x)) (1 + w2)
              (the sublayers read x itself; the norm sits on their OUTPUT; l1, l2 are per-channel layer scales)
  N           RMS norm, y / sqrt(mean(y^2) + eps)
  mixer       "attention": softmax attention over the last W tokens plus one averaged key / value per block of P tokens
              that ends before they begin, a sink logit in the denominator, a sigmoid gate per head; keys and values
              may be another layer's.  "mamba2": a state-space recurrence with one scalar decay per head and token.
              "delta": the gated delta rule with one scalar decay per head and token.
  ff          down(silu(gate x) * up x)
  output      logits = c * tanh(E (N(x) (1 + w_f)) / c)
"""
import math
from typing import Dict, List, Optional

import torch


# ----------------------------------------------------------------------------------- small pieces
def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """The weight is stored around zero."""
    return unit_rms(x, eps) * (1.0 + w)


def causal_conv(u: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """u [T, C], w [C, taps]; the LAST tap multiplies the current token, tap taps-1-k the token k steps back."""
    T, C = u.shape
    taps = w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for k in range(taps):
            if t - k >= 0:
                y[t] += w[:, taps - 1 - k] * u[t - k]
    if bias is not None:
        y = y + bias
    return y


# ----------------------------------------------------------------------------------- rotation
def scaled_frequencies(dims: int, base: float, scaling: Optional[dict]) -> (torch.Tensor, float):
    """Frequencies f_i, i < dims / 2, and the factor on cos and sin.  With scaling {factor, original, fast, slow}:
    a feature pair that turns more than `fast` times over `original` positions keeps its frequency, one that turns fewer
    than `slow` times has it divided by `factor`, with a linear ramp over the pair index between the two."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def pair_index(turns: float) -> float:
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_index(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_index(float(scaling["slow"]))), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(half)], dtype=torch.float64)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_half(x: torch.Tensor, dims: int, freqs: torch.Tensor, mag: float) -> torch.Tensor:
    """x [T, H, d]: feature i < dims / 2 is paired with feature i + dims / 2; the rest pass unchanged."""
    T = x.shape[0]
    half = dims // 2
    ang = torch.arange(T, dtype=torch.float64)[:, None] * freqs[None, :].to(torch.float64)
    c, s = (torch.cos(ang) * mag).to(x.dtype)[:, None, :], (torch.sin(ang) * mag).to(x.dtype)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    out = x.clone()
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


# ----------------------------------------------------------------------------------- mixers
def pooled_window_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: int, pool: int,
                            sink: Optional[torch.Tensor]) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv].  Token i sees j with 0 <= i - j < window and, for every
    block b of `pool` tokens whose last token b pool + pool - 1 <= i - window, the block's mean key with its mean value.
    exp(sink_h) sits in the denominator without a value."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    nblk = T // pool if pool > 0 else 0
    if nblk:
        kp = k[: nblk * pool].reshape(nblk, pool, G, -1).mean(1)
        vp = v[: nblk * pool].reshape(nblk, pool, G, -1).mean(1)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            lo = max(0, i - window + 1) if window > 0 else 0
            keys, vals = [k[lo: i + 1, g]], [v[lo: i + 1, g]]
            if pool > 0 and window > 0:
                seen = [b for b in range(nblk) if b * pool + pool - 1 <= i - window]
                if seen:
                    keys.insert(0, kp[seen, g])
                    vals.insert(0, vp[seen, g])
            kk, vv = torch.cat(keys), torch.cat(vals)
            s = (kk @ q[i, h]) * scale
            m = s.max() if sink is None else torch.maximum(s.max(), sink[h].to(s.dtype))
            e = torch.exp(s - m)
            den = e.sum() + (torch.exp(sink[h].to(s.dtype) - m) if sink is not None else 0.0)
            out[i, h] = (e[:, None] * vv).sum(0) / den
    return out


def attention_keys_values(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mx: dict, eps: float):
    """Keys after their norm and rotation, values after their unit norm: what a cache holds.  [T, G, d], [T, G, dv]."""
    T = h.shape[0]
    G, d, dv = mx["kv_heads"], mx["dim"], mx["vdim"]
    rot = mx.get("rot")
    k = (h @ w[p + "k"].T + w[p + "k.b"]).view(T, G, d)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).view(T, G, dv)
    k = unit_rms(k, eps) * w[p + "k.norm"]
    if rot:
        f, mag = scaled_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        k = rotate_half(k, rot["dims"], f, mag)
    return k, unit_rms(v, eps)


def attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mx: dict, eps: float, kv) -> torch.Tensor:
    """kv: (keys, values) as attention_keys_values gives them, of this layer or of the layer it borrows from."""
    T = h.shape[0]
    H, d, dv = mx["heads"], mx["dim"], mx["vdim"]
    rot = mx.get("rot")
    q = (h @ w[p + "q"].T + w[p + "q.b"]).view(T, H, d)
    q = unit_rms(q, eps) * w[p + "q.norm"]
    if rot:
        f, mag = scaled_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q = rotate_half(q, rot["dims"], f, mag)
    mask = mx.get("mask") or {}
    o = pooled_window_attention(q, kv[0], kv[1], float(mx["scale"]), int(mask.get("size", 0)), int(mask.get("pool", 0)),
                                w.get(p + "sink"))
    gate = torch.sigmoid(h @ w[p + "g"].T)                    # [T, H]
    return (o * gate[:, :, None]).reshape(T, H * dv) @ w[p + "o"].T


def state_space_recurrence(x: torch.Tensor, B: torch.Tensor, C: torch.Tensor, dt: torch.Tensor, rate: torch.Tensor,
                           skip: Optional[torch.Tensor]) -> torch.Tensor:
    """x [T, H, dv], B, C [T, G, N], dt [T, H] (step sizes, already positive), rate [H] -> y [T, H, dv]:
    S_t = exp(-rate dt_t) S_{t-1} + dt_t B_t x_t^T,  y_t = S_t^T C_t + skip x_t."""
    T, H, dv = x.shape
    G, N = B.shape[1], B.shape[2]
    y = torch.zeros(T, H, dv, dtype=x.dtype)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(N, dv, dtype=x.dtype)
        for t in range(T):
            S = torch.exp(-rate[hd] * dt[t, hd]) * S + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S.T @ C[t, g] + (skip[hd] * x[t, hd] if skip is not None else 0.0)
    return y


def gated_delta_rule(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, beta: torch.Tensor, decay: torch.Tensor) -> torch.Tensor:
    """q, k [T, G, d], v [T, H, dv], beta, decay [T, H] -> o [T, H, dv]: S <- decay S; u = beta (v - S^T k); S <- S + k u^T;
    o = S^T q, the read-out after the write."""
    T, H, dv = v.shape
    G, d = q.shape[1], q.shape[2]
    o = torch.zeros(T, H, dv, dtype=v.dtype)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(d, dv, dtype=v.dtype)
        for t in range(T):
            S = decay[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            o[t, hd] = S.T @ q[t, g]
    return o


def unit_vectors(x: torch.Tensor) -> torch.Tensor:
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def gated_group_norm(y: torch.Tensor, z: torch.Tensor, w: torch.Tensor, parts: int, eps: float) -> torch.Tensor:
    """y, z [T, D]: the gate silu(z) first, then the RMS norm of each of `parts` equal parts of the row, then the weight."""
    T, D = y.shape
    g = y * silu(z)
    return unit_rms(g.view(T, parts, D // parts), eps).reshape(T, D) * w


def mamba2_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mx: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, dv, N, G = mx["heads"], mx["vdim"], mx["state"], mx["groups"]
    inner = H * dv
    proj = h @ w[p + "in"].T
    z = proj[:, :inner]
    xbc = silu(causal_conv(proj[:, inner: 2 * inner + 2 * G * N], w[p + "conv"], w[p + "conv.b"]))
    dt = softplus(proj[:, 2 * inner + 2 * G * N:] + w[p + "dt_bias"])          # [T, H]
    x = xbc[:, :inner].view(T, H, dv)
    B = xbc[:, inner: inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    y = state_space_recurrence(x, B, C, dt, torch.exp(w[p + "A_log"]), w[p + "D"])
    y = gated_group_norm(y.reshape(T, inner), z, w[p + "norm"], int(mx.get("norm_groups", 1)), eps)
    return y @ w[p + "o"].T


def delta_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mx: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, d, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = silu(causal_conv(h @ w[p + "q"].T, w[p + "q.conv"])).view(T, G, d)
    k = silu(causal_conv(h @ w[p + "k"].T, w[p + "k.conv"])).view(T, G, d)
    v = silu(causal_conv(h @ w[p + "v"].T, w[p + "v.conv"])).view(T, H, dv)
    q = unit_vectors(q) * d ** -0.5
    k = unit_vectors(k)
    beta = torch.sigmoid(h @ w[p + "b"].T)                                       # [T, H]
    decay = torch.exp(-torch.exp(w[p + "A_log"]) * softplus(h @ w[p + "a"].T + w[p + "dt_bias"]))
    o = gated_delta_rule(q, k, v, beta, decay)
    o = unit_rms(o, eps) * w[p + "norm"]
    o = o.reshape(T, H * dv) * silu(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def dense_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


# ----------------------------------------------------------------------------------- the model
def forward(config: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64, streams: Optional[list] = None):
    """Logits [T, vocab] of one sequence; `streams` (a list) receives the residual stream after every layer."""
    w = {n: t.to(dtype) if t.is_floating_point() else t for n, t in weights.items()}
    eps = float(config["norm"]["eps"])
    m = float(config.get("residual_mult", 1.0))
    x = w["embed"][torch.tensor(tokens)] * float(config["embedding"]["scale"])
    kv = {}
    for i, spec in enumerate(config["layers"]):
        p, mx = f"l{i}.mix.", spec["mixer"]
        if spec["type"] == "attention":
            src = mx.get("kv_from")
            kv[i] = kv[src] if src is not None else attention_keys_values(x, w, p, mx, eps)
            y = attention_mixer(x, w, p, mx, eps, kv[i])
        elif spec["type"] == "mamba2":
            y = mamba2_mixer(x, w, p, mx, eps)
        elif spec["type"] == "delta":
            y = delta_mixer(x, w, p, mx, eps)
        else:
            raise ValueError(spec["type"])
        x = x + m * w[f"l{i}.ls1"] * offset_rms_norm(y, w[f"l{i}.norm1"], eps)
        if spec.get("mlp") is not None:
            x = x + m * w[f"l{i}.ls2"] * offset_rms_norm(dense_ff(x, w, f"l{i}.mlp."), w[f"l{i}.norm2"], eps)
        if streams is not None:
            streams.append(x.clone())
    logits = offset_rms_norm(x, w["final.norm"], eps) @ w["embed"].T
    cap = config.get("logit_softcap")
    if cap:
        logits = float(cap) * torch.tanh(logits / float(cap))
    return logits


def greedy(config: dict, weights: Dict[str, torch.Tensor], prompt: List[int], n: int) -> List[int]:
    """n tokens, each the arg-max of the whole-sequence logits at the last position (the lowest id on a tie)."""
    toks, out = list(prompt), []
    for _ in range(n):
        nxt = int(torch.argmax(forward(config, weights, toks)[-1]))
        out.append(nxt)
        toks.append(nxt)
    return out
