"""Checks of single Gatarax mechanisms against the oracle's functions (oracle/gatarax_ref.py), written once for any ops
object: the HIP kernels on the GPU (test_gatarax_gpu.py) and the CPU stand-ins (test_gatarax_cpu.py).  Every case builds
the request table, positions and state pool by hand, so that slots, pages and cuts are the case's to choose."""
import math

import torch

from oracle import gatarax_ref as ref
from verozen_cases import KVSetup, Table, _bf, _close, _tol


def _segs(b, decode):
    return {} if decode else dict(tok_req=b["tok_req"], seg_start=b["seg_start"], seg_len=b["seg_len"])


# ------------------------------------------------------------------------------------------- norm and residual sum
def check_offset_norm_and_branch_add(ops, device, dtype, T=7, D=48, eps=1e-5):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(T, D, generator=g) * 3
    w = _bf(0.1 * torch.randn(D, generator=g))
    h = ops.offset_rmsnorm(x.to(device), w.to(dtype).to(device), eps, 1.0)
    assert h.dtype == dtype
    _close(h, ref.offset_rms_norm(x.double(), w, eps), _tol(dtype), "norm with a weight stored around zero")
    a, b, f = (_bf(torch.randn(T, D + 3, generator=g) * s)[:, 1: 1 + D] for s in (2.0, 0.3, 1.0))
    wa, wb = (_bf(1 + 0.1 * torch.randn(D, generator=g)) for _ in range(2))
    dev = lambda t: t.to(dtype).to(device)
    # two normed branches, half their sum, a dense third
    xd = x.clone().to(device)
    ops.branch_residual_add(xd, dev(a), dev(wa), dev(b), dev(wb), 0.5, f=dev(f), eps=eps)
    _close(xd, x.double() + 0.5 * (ref.unit_rms(a, eps) * wa + ref.unit_rms(b, eps) * wb) + f, 2e-6, "two normed branches and a dense one")
    # one plain branch and a weighted sum of picked rows
    big = _bf(torch.randn(3 * T + 2, D, generator=g))
    rows = torch.randint(0, 3 * T + 2, (T, 3), generator=g, dtype=torch.int32)
    coef = torch.rand(T, 3, generator=g)
    xd = x.clone().to(device)
    ops.branch_residual_add(xd, dev(a), None, f=dev(big), rows=rows.to(device), coef=coef.to(device), eps=eps)
    _close(xd, x.double() + a + (coef.double()[:, :, None] * big[rows.long()]).sum(1), 2e-6, "a plain branch and a weighted sum of rows")
    # a plain branch alone
    xd = x.clone().to(device)
    ops.branch_residual_add(xd, dev(a), None, eps=eps)
    _close(xd, x.double() + a, 2e-6, "a plain branch alone")


def check_gates_and_activations(ops, device, dtype, T=6, H=3, dv=20, eps=1e-5):
    g = torch.Generator().manual_seed(8)
    o = torch.randn(T, H, dv, generator=g) * 5
    gate = _bf(torch.randn(T, H * dv + 7, generator=g))
    w = _bf(1 + 0.1 * torch.randn(dv, generator=g))
    want = (ref.unit_rms(o.double(), eps) * w).reshape(T, H * dv) * torch.sigmoid(gate[:, 3: 3 + H * dv])
    got = ops.head_rmsnorm_gate_act(o.to(device), w.to(dtype).to(device), gate.to(dtype).to(device)[:, 3: 3 + H * dv], eps, dtype, "sigmoid")
    _close(got, want, _tol(dtype), "head norm with a sigmoid gate")
    # all heads as one: the norm runs over the whole row
    wide = _bf(1 + 0.1 * torch.randn(H * dv, generator=g))
    want = ref.unit_rms(o.double().reshape(T, 1, H * dv), eps).reshape(T, H * dv) * wide * torch.sigmoid(gate[:, : H * dv])
    got = ops.head_rmsnorm_gate_act(o.to(device).view(T, 1, H * dv), wide.to(dtype).to(device), gate.to(dtype).to(device)[:, : H * dv], eps,
                                    dtype, "sigmoid")
    _close(got, want, _tol(dtype), "one norm over all heads with a sigmoid gate")
    z = gate.to(dtype).to(device)[:, 2: 2 + 31]
    _close(ops.activation(z, "silu"), ref.silu(gate[:, 2: 2 + 31]), _tol(dtype), "silu")
    _close(ops.activation(z, "relu2"), ref.relu_squared(gate[:, 2: 2 + 31]), _tol(dtype), "squared relu")
    assert float(ops.activation(z, "relu2").min()) == 0.0


# ------------------------------------------------------------------------------------------- short convolutions
def run_conv(ops, device, dtype, u, w1, w2, cuts, residual, act, slot=2, decode_tail=0, state=None, pad=3):
    """One sequence cut into portions (the last decode_tail single tokens as decode steps without segment arrays); the
    input rows sit inside a wider tensor."""
    T, C = u.shape
    taps = w1.shape[1]
    tab = Table(device)
    tab.req_to_state[4] = slot
    if state is None:
        state = torch.full((5, taps - 1, C), 55.0, dtype=torch.float32, device=device)      # stale: position 0 must not read it
    wide = torch.zeros(T, C + 2 * pad, dtype=dtype)
    wide[:, pad: pad + C] = u.to(dtype)
    wide = wide.to(device)
    outs, at = [[], []], 0
    for n in cuts:
        decode = at >= T - decode_tail and n == 1
        b = tab.batch([(4, at, n)])
        y = ops.causal_conv(wide[at: at + n, pad: pad + C], w1.to(dtype).to(device), state, tab.req_to_state, b["req_pool_indices"],
                            b["positions"], w2=w2.to(dtype).to(device) if w2 is not None else None, residual=residual, act=act,
                            **_segs(b, decode))
        ys = (y,) if w2 is None else y
        for o, part in zip(outs, ys):
            o.append(part.cpu())
        at += n
    assert at == T
    return [torch.cat(o) for o in outs if o], state


def check_conv(ops, device, dtype, taps=4, C=40, T=37, cuts=(37,), residual=False, act="none", two=False, decode_tail=0):
    g = torch.Generator().manual_seed(10 + taps)
    u = _bf(torch.randn(T, C, generator=g))
    w1 = _bf(torch.randn(C, taps, generator=g) * 0.5)
    w2 = _bf(torch.randn(C, taps, generator=g) * 0.5) if two else None
    got, state = run_conv(ops, device, dtype, u, w1, w2, cuts, residual, act, decode_tail=decode_tail)
    for y, w in zip(got, (w1, w2)):
        want = ref.causal_conv(u, w) + (u if residual else 0.0)
        if act == "silu":
            want = ref.silu(want)
        _close(y, want, _tol(dtype), f"convolution of {taps} taps cut into {list(cuts)[:8]}")
    if taps > 1:
        _close(state[2], u[T - (taps - 1):] if T >= taps - 1 else torch.cat([torch.zeros(taps - 1 - T, C, dtype=torch.float64), u]),
               1e-6, "the state holds the last inputs")
        assert float(state[1].min()) == 55.0 and float(state[3].min()) == 55.0, "only the sequence's slot is written"


def check_conv_planted(ops, device, dtype):
    """One input spike: the token taps - 1 later still hears it through the oldest tap, the next one does not -- with the
    spike on either side of a cut, in the state of a decode step, and at position 0."""
    taps, C = 4, 8
    w = torch.zeros(C, taps, dtype=torch.float64)
    w[:, 0], w[:, 3] = 0.5, 0.25
    for spike in (0, 5, 63):
        T = spike + 8
        u = torch.zeros(T, C, dtype=torch.float64)
        u[spike, 2] = 4.0
        for cuts, tail in (([T], 0), ([spike + 1, T - spike - 1], 0), ([spike + 3, 1, T - spike - 4], 0), ([spike + 2] + [1] * 6, 6),
                           ([spike + 2, 2, 2, 2], 0)):
            (y,), _ = run_conv(ops, device, dtype, u, w, None, cuts, False, "none", decode_tail=tail)
            assert abs(float(y[spike, 2]) - 1.0) < 1e-6 and abs(float(y[spike + 3, 2]) - 2.0) < 1e-6, (spike, cuts)
            y[spike, 2] = 0
            y[spike + 3, 2] = 0
            assert float(y.abs().max()) == 0.0, (spike, cuts)


def check_conv_batch(ops, device, dtype):
    """Three sequences of unequal length in one call, each with its own slot, against each alone; then all three go on by a
    single token in a decode step."""
    g = torch.Generator().manual_seed(12)
    taps, C = 3, 24
    w = _bf(torch.randn(C, taps, generator=g))
    us = [_bf(torch.randn(n, C, generator=g)) for n in (9, 2, 14)]
    first = [5, 1, 9]
    tab = Table(device)
    for row, slot in ((0, 3), (1, 1), (2, 2)):
        tab.req_to_state[row] = slot
    state = torch.full((4, taps - 1, C), 9.0, dtype=torch.float32, device=device)
    b = tab.batch([(r, 0, first[r]) for r in range(3)])
    y = ops.causal_conv(torch.cat([u[:n] for u, n in zip(us, first)]).to(dtype).to(device), w.to(dtype).to(device), state,
                        tab.req_to_state, b["req_pool_indices"], b["positions"], residual=True, **_segs(b, False)).cpu()
    at = 0
    for u, n in zip(us, first):
        _close(y[at: at + n], (ref.causal_conv(u, w) + u)[:n], _tol(dtype), "a sequence of a batch")
        at += n
    b = tab.batch([(r, first[r], 1) for r in range(3)])
    y = ops.causal_conv(torch.stack([u[n] for u, n in zip(us, first)]).to(dtype).to(device), w.to(dtype).to(device), state,
                        tab.req_to_state, b["req_pool_indices"], b["positions"], residual=True).cpu()
    for r, (u, n) in enumerate(zip(us, first)):
        _close(y[r], (ref.causal_conv(u, w) + u)[n], _tol(dtype), "a decode step of a batch")


# ------------------------------------------------------------------------------------------- windowed attention with a sink
def run_window_attention(ops, device, dtype, q, kn, v, scale, window, cuts, page=1, decode_tail=0, sink=0.0, pad_q=0, splits=1):
    T, H, d = q.shape
    G = kn.shape[1]
    kv = KVSetup(device, dtype, kn, v, page=page)
    bq = ops.window_attention_block_tokens(H, G, d, v.shape[-1], dtype)
    wide = torch.zeros(T, H * d + pad_q, dtype=dtype)
    wide[:, : H * d] = q.reshape(T, H * d).to(dtype)
    qd = wide.to(device)[:, : H * d].view(T, H, d)
    if qd.stride(0) % 8:
        qd = qd.contiguous()
    sk = None if sink is None else torch.full((H,), float(sink), dtype=torch.float32, device=device)
    outs, at = [], 0
    for n in cuts:
        decode = at >= T - decode_tail and n == 1
        b = kv.tab.batch([(kv.row, at, n)])
        o = torch.zeros((n, H, v.shape[-1]), dtype=dtype, device=device)
        blocks = None
        if not decode:
            blocks = torch.tensor([[s, min(bq, n - s)] for s in range(0, n, bq)], dtype=torch.int32, device=device)
        ops.window_attention(qd[at:at + n], kv.k_cache, kv.v_cache, o, kv.tab.req_to_token, b["req_pool_indices"], b["positions"], sk,
                             window, scale, tok_req=None if decode else b["tok_req"], blocks=blocks, max_run=bq,
                             num_splits=splits if decode else 1)
        outs.append(o.cpu())
        at += n
    return torch.cat(outs)


def check_window_attention(ops, device, dtype, H=4, G=2, d=32, dv=32, T=150, window=40, cuts=(150,), page=1, decode_tail=0, pad_q=0,
                           splits=1):
    g = torch.Generator().manual_seed(3)
    q = _bf(torch.randn(T, H, d, generator=g))
    kn = _bf(torch.randn(T, G, d, generator=g))
    v = _bf(torch.randn(T, G, dv, generator=g))
    scale = 1.7 / math.sqrt(d)
    want = ref.window_sink_attention(q, kn, v, scale, window)
    got = run_window_attention(ops, device, dtype, q, kn, v, scale, window, cuts, page=page, decode_tail=decode_tail, pad_q=pad_q,
                               splits=splits)
    _close(got, want, 2e-5 if dtype == torch.float32 else 1.5e-2, f"window attention ({H}/{G} heads of {d}/{dv}) cut into {list(cuts)[:6]}, pages of {page}")


def check_window_attention_planted(ops, device, dtype):
    """Scores are zero except where a query and a key are made to meet (score 16): the key exactly window - 1 back is
    seen, the one window back is not, also across a page's border and in decode steps; a far key is out of reach; and a row
    that sees only zero scores gives its n keys the weight 1 / (n + 1) each: the sink counts as one more."""
    H, G, d, T, W = 2, 1, 32, 300, 56
    j1, j3 = 120, 128 - (W - 1)            # j1 and j1 + 1 are asked for from j1 + W - 1 and the token after; j3 from 128 and 129
    a = j1 + W - 1
    q = torch.zeros(T, H, d, dtype=torch.float64)
    kn = torch.zeros(T, G, d, dtype=torch.float64)
    v = torch.zeros(T, G, d, dtype=torch.float64)
    for j, col in ((2, 0), (j1, 1), (j1 + 1, 2), (j3, 3), (T - 1, 4)):
        kn[j, 0, col] = 4.0
        v[j, 0, col] = 1.0 + col

    def ask(i, cols):
        q[i] = 0
        for c in cols:
            q[i, :, c] = 4.0
    ask(a, [1, 2])         # a - j1 = window - 1: seen; j1 + 1 seen too
    ask(a + 1, [1, 2])     # j1 is a whole window back: gone; j1 + 1 still seen
    ask(128, [3])          # 128 - j3 = window - 1: seen, across the borders at 64 and 128
    ask(129, [3])          # gone
    ask(T - 1, [0, 4])     # the far key 2 is out of reach, its own key is seen
    hot = math.exp(16.0)
    for cuts, tail in (([T], 0), ([a - 1, 1, 1, 1, T - a - 2], 0), ([128, 1, 1, a - 130, T - a], 0), ([a, 1, 1, T - a - 2], 0),
                       ([T - 2, 1, 1], 2), ([a - 5] + [1] * 10 + [T - a - 5], 0)):
        assert sum(cuts) == T
        for page in (1, 64):
            got = run_window_attention(ops, device, dtype, q, kn, v, 1.0, W, cuts, page=page, decode_tail=tail,
                                       splits=3 if page == 64 else 1).double()
            tol = 1e-5 if dtype == torch.float32 else 1e-2
            den = 2 * hot + (W - 2) + 1                      # two hot keys, the cold rest of the window, the sink
            assert abs(float(got[a, 0, 1]) - 2.0 * hot / den) < tol and abs(float(got[a, 1, 2]) - 3.0 * hot / den) < tol, (cuts, page)
            den = hot + (W - 1) + 1
            assert abs(float(got[a + 1, 0, 1])) < 1e-6 and abs(float(got[a + 1, 0, 2]) - 3.0 * hot / den) < tol, (cuts, page)
            assert abs(float(got[128, 1, 3]) - 4.0 * hot / den) < tol and abs(float(got[129, 1, 3])) < 1e-6, (cuts, page)
            assert abs(float(got[T - 1, 0, 0])) < 1e-6 and abs(float(got[T - 1, 1, 4]) - 5.0 * hot / den) < tol, (cuts, page)
            # token 5 sees six keys of score zero, one of which (key 2) holds 1.0 in column 0: 1 / (6 + 1)
            assert abs(float(got[5, 0, 0]) - 1.0 / 7.0) < tol, (cuts, page)
            assert float(got[0].abs().max()) == 0.0 and float(got[1].abs().max()) == 0.0
    # without the sink the same row gives 1 / 6
    got = run_window_attention(ops, device, dtype, q, kn, v, 1.0, W, [T], sink=None).double()
    assert abs(float(got[5, 0, 0]) - 1.0 / 6.0) < (1e-5 if dtype == torch.float32 else 1e-2)
    # a window wider than the sequence (and no window at all): the far key 2 is one hot key among hundreds for the last token,
    # whole, cut, and decoded over key ranges
    for window in (T + 50, 0):
        for cuts, tail, splits in (([T], 0, 1), ([3, 2, T - 6, 1], 0, 1), ([T - 1, 1], 1, 4)):
            got = run_window_attention(ops, device, dtype, q, kn, v, 1.0, window, cuts, page=64, decode_tail=tail, splits=splits).double()
            den = 2 * hot + (T - 2) + 1
            tol = 1e-5 if dtype == torch.float32 else 1e-2
            assert abs(float(got[T - 1, 0, 0]) - 1.0 * hot / den) < tol and abs(float(got[T - 1, 1, 4]) - 5.0 * hot / den) < tol, (window, cuts)


# ------------------------------------------------------------------------------------------- gated delta rule
def run_delta_rule(ops, device, dtype, q, k, v, beta_logits, z, rate_bias, rate_log, cuts, q_scale=1.0, slot=2, decode_tail=0, state=None):
    T, G, dk = q.shape
    H, dv = v.shape[1], v.shape[2]
    tab = Table(device)
    tab.req_to_state[4] = slot
    if state is None:
        state = torch.full((5, H, dk, dv), 77.0, dtype=torch.float32, device=device)     # stale: position 0 must not read it
    qd, kd = q.float().to(device), k.float().to(device)
    vd = v.to(dtype).to(device)
    wide = torch.zeros(T, H + 5, dtype=dtype)
    wide[:, 2: 2 + H] = beta_logits.to(dtype)
    bd = wide.to(device)[:, 2: 2 + H]
    zd = z.float().to(device)
    outs, at = [], 0
    for n in cuts:
        decode = at >= T - decode_tail and n == 1
        b = tab.batch([(4, at, n)])
        o = torch.empty((n, H, dv), dtype=torch.float32, device=device)
        ops.gated_delta_rule(qd[at:at + n], kd[at:at + n], vd[at:at + n], bd[at:at + n], zd[at:at + n], rate_bias.float().to(device),
                             rate_log.float().to(device), o, state, tab.req_to_state, b["req_pool_indices"], b["positions"], q_scale,
                             **_segs(b, decode))
        outs.append(o.cpu())
        at += n
    assert at == T
    return torch.cat(outs), state


def check_delta_rule(ops, device, dtype, H=4, G=2, dk=12, dv=20, T=45, cuts=(45,), decode_tail=0):
    g = torch.Generator().manual_seed(2)
    q = ref.unit_vectors(torch.randn(T, G, dk, generator=g).double()).float().double()
    k = ref.unit_vectors(torch.randn(T, G, dk, generator=g).double()).float().double()
    v = _bf(torch.randn(T, H, dv, generator=g))
    beta_logits = _bf(torch.randn(T, H, generator=g))
    z = torch.randn(T, H * dk, generator=g).float().double()
    rate_bias = _bf(torch.randn(H * dk, generator=g) - 1.0)
    rate_log = _bf(torch.randn(H, generator=g) * 0.5)
    decay = torch.exp(-torch.exp(rate_log)[None, :, None] * torch.nn.functional.softplus(z + rate_bias).reshape(T, H, dk))
    want = ref.gated_delta_rule(q * 0.37, k, v, torch.sigmoid(beta_logits), decay)
    got, _ = run_delta_rule(ops, device, dtype, q, k, v, beta_logits, z, rate_bias, rate_log, cuts, q_scale=0.37, decode_tail=decode_tail)
    _close(got, want, 5e-5, f"gated delta rule ({H}/{G} heads of {dk}/{dv}) cut into {list(cuts)[:6]}")


def check_delta_rule_planted(ops, device, dtype):
    """With a decay of (almost) one and beta (almost) one, a value written under a key 600 tokens back is read back in full;
    writing another value under the same key REPLACES it (the rule subtracts what the key already recalls); a head whose
    decay is small has forgotten; a sequence's first token starts from zero whatever its slot held."""
    H, G, dk, dv, T = 2, 1, 8, 8, 640
    q = torch.zeros(T, G, dk, dtype=torch.float64)
    k = torch.zeros(T, G, dk, dtype=torch.float64)
    v = torch.zeros(T, H, dv, dtype=torch.float64)
    k[3, 0, 1] = 1.0
    v[3, :, 5] = 2.0
    q[4, 0, 1] = 1.0
    q[610, 0, 1] = 1.0
    k[620, 0, 1] = 1.0
    v[620, :, 5] = -3.0
    q[T - 1, 0, 1] = 1.0
    beta_logits = torch.full((T, H), 30.0, dtype=torch.float64)
    z = torch.zeros(T, H * dk, dtype=torch.float64)
    rate_bias = torch.zeros(H * dk, dtype=torch.float64)
    rate_log = torch.tensor([-40.0, 0.0], dtype=torch.float64)        # head 0 keeps everything, head 1 decays by exp(-log 2) a token
    for cuts, tail in (([T], 0), ([4, 2, 600, 34], 0), ([5] + [127] * 5, 0), ([620, 1, 19], 0), ([630] + [1] * 10, 10)):
        got, state = run_delta_rule(ops, device, dtype, q, k, v, beta_logits, z, rate_bias, rate_log, cuts, decode_tail=tail)
        assert abs(float(got[4, 0, 5]) - 2.0) < 1e-5 and abs(float(got[4, 1, 5]) - 1.0) < 1e-5, cuts
        assert abs(float(got[610, 0, 5]) - 2.0) < 1e-5 and abs(float(got[610, 1, 5])) < 1e-30, cuts
        assert abs(float(got[T - 1, 0, 5]) + 3.0) < 1e-5, f"{cuts}: the second write replaces the first"
        assert float(got[:3].abs().max()) == 0.0, cuts
        assert abs(float(state[2, 0, 1, 5]) + 3.0) < 1e-5 and float(state[1].min()) == 77.0, "only the sequence's slot is written"


# ------------------------------------------------------------------------------------------- mixture
def check_router_softmax(ops, device, E=12, n_groups=4, keep=2, top=3, T=64):
    g = torch.Generator().manual_seed(4)
    logits = (torch.randn(T, E, generator=g) * 2).float()
    scores = torch.softmax(logits.double(), -1)
    chosen, weights = ref.route(scores, top, n_groups, keep)
    ids, wt = ops.moe_route_scores(logits.to(device), None, top, n_groups, keep, 1.0, score_fn="softmax", group_best=1, renorm=False)
    assert ids.dtype == torch.int32 and wt.dtype == torch.float32
    ids, wt = ids.cpu(), wt.cpu()
    for t in range(T):
        assert sorted(ids[t].tolist()) == sorted(chosen[t].tolist()), f"token {t}: {ids[t].tolist()} for {chosen[t].tolist()}"
        for e, c in zip(chosen[t].tolist(), weights[t].tolist()):
            assert abs(float(wt[t, ids[t].tolist().index(e)]) - c) < 1e-6
    # a group is judged by its best member alone: one strong expert beats two middling ones
    lg = torch.full((1, 6), -5.0)
    lg[0, 0] = 3.0                      # group 0: one strong, one weak
    lg[0, 2], lg[0, 3] = 2.0, 2.0       # group 1: two middling (their sum would win)
    ids, _ = ops.moe_route_scores(lg.to(device), None, 2, 3, 1, 1.0, score_fn="softmax", group_best=1, renorm=False)
    assert sorted(ids.cpu()[0].tolist()) == [0, 1]


def check_gated_experts(ops, device, dtype, T=37, D=48, ff=40, E=5, top=2, wide_ok=False, tiled_ok=False, block=None):
    g = torch.Generator().manual_seed(6)
    h = _bf(torch.randn(T, D, generator=g))
    gate_up = _bf(torch.randn(E, 2 * ff, D, generator=g) * D ** -0.5)
    down = _bf(torch.randn(E, D, ff, generator=g) * ff ** -0.5)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    plan = ops.moe_align(ids.to(device), E, wide_ok=wide_ok, tiled_ok=tiled_ok)
    assert block is None or plan.block == block
    a = ops.silu_and_mul(ops.moe_grouped_linear(h.to(dtype).to(device), gate_up.to(dtype).to(device), plan, gather=True, gelu=False))
    y = ops.moe_grouped_linear(a, down.to(dtype).to(device), plan, gather=False, gelu=False)
    rows = plan.rows.cpu().long()
    want = torch.stack([torch.stack([(ref.silu(h[t] @ gate_up[int(e), :ff].T) * (h[t] @ gate_up[int(e), ff:].T)) @ down[int(e)].T
                                     for e in ids[t]]) for t in range(T)])
    _close(y.cpu()[rows], want, 2e-5 if dtype == torch.float32 else 3e-2, "silu-gated experts over sorted blocks")
