"""Checks of single Fudonex mechanisms against the oracle's functions (oracle/fudonex_ref.py), written once for any ops
object: the HIP kernels on the GPU (test_fudonex_gpu.py) and the CPU stand-ins (test_fudonex_cpu.py).  Every case builds
the request table, positions and state pool by hand, so that slots, pages and cuts are the case's to choose."""
import math

import torch

from oracle import fudonex_ref as ref
from verozen_cases import KVSetup, Table, _bf, _close, _tol


def _segs(b, decode):
    return {} if decode else dict(tok_req=b["tok_req"], seg_start=b["seg_start"], seg_len=b["seg_len"])


# ------------------------------------------------------------------------------------------- norms
def check_output_norm_add(ops, device, dtype, T=7, D=48, eps=1e-5, mult=0.5):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(T, D, generator=g) * 3
    y = _bf(torch.randn(T, D + 5, generator=g) * 4)[:, 2: 2 + D]
    w = _bf(0.1 * torch.randn(D, generator=g))
    ls = _bf(1 + 0.3 * torch.randn(D, generator=g))
    dev = lambda t: t.to(dtype).to(device)
    wide = torch.zeros(T, D + 5, dtype=dtype)
    wide[:, 2: 2 + D] = y.to(dtype)
    xd = x.clone().to(device)
    h = ops.rmsnorm_residual_add(xd, wide.to(device)[:, 2: 2 + D], dev(w), eps, offset=1.0, layer_scale=dev(ls), mult=mult)
    want = x.double() + mult * ls * ref.offset_rms_norm(y, w, eps)
    _close(xd, want, 2e-6, "normed output with a layer scale added to the stream")
    assert h.dtype == dtype
    _close(h, want, _tol(dtype), "the stream's copy in the activation dtype")
    # the plain form still does what it did: no offset, no layer scale
    xd = x.clone().to(device)
    ops.rmsnorm_residual_add(xd, wide.to(device)[:, 2: 2 + D], dev(ls), eps)
    _close(xd, x.double() + ref.unit_rms(y, eps) * ls, 2e-6, "plain normed residual add")


def check_gated_group_norm(ops, device, dtype, T=6, D=60, eps=1e-5, parts_list=(1, 3, 60)):
    g = torch.Generator().manual_seed(8)
    y = torch.randn(T, D, generator=g) * 5
    z = _bf(torch.randn(T, D + 7, generator=g))
    w = _bf(1 + 0.1 * torch.randn(D, generator=g))
    for parts in parts_list:
        got = ops.gated_group_rmsnorm(y.to(device), z.to(dtype).to(device)[:, 3: 3 + D], w.to(dtype).to(device), parts, eps)
        assert got.dtype == dtype
        _close(got, ref.gated_group_norm(y.double(), z[:, 3: 3 + D], w, parts, eps), _tol(dtype), f"gate, then norm in {parts} parts")
    # gated first, normed after: a row whose gate is tiny everywhere still leaves the norm at full size
    zs = torch.full((1, D), -12.0, dtype=torch.float64)
    got = ops.gated_group_rmsnorm(y[:1].to(device), zs.to(dtype).to(device), torch.ones(D, dtype=dtype, device=device), 1, 0.0)
    assert abs(float(got.double().pow(2).mean().sqrt()) - 1.0) < (1e-4 if dtype == torch.float32 else 2e-2)
    # rows longer than one pass of the workgroup keeps in registers
    D2 = 2304
    y2, z2 = torch.randn(2, D2, generator=g), _bf(torch.randn(2, D2, generator=g))
    w2 = _bf(1 + 0.1 * torch.randn(D2, generator=g))
    got = ops.gated_group_rmsnorm(y2.to(device), z2.to(dtype).to(device), w2.to(dtype).to(device), 1, eps)
    _close(got, ref.gated_group_norm(y2.double(), z2, w2, 1, eps), _tol(dtype), "a long row")


# ------------------------------------------------------------------------------------------- rotation
def check_scaled_frequencies():
    """The package's frequency table against the oracle's, also where the two ends of the ramp meet or cross."""
    from sglang_custom_amd.layers.rotary_embedding import scaled_pair_inv_freq

    for dims, base, sc in ((8, 500.0, dict(factor=4.0, original=16, fast=2.0, slow=0.5)), (40, 30000.0, dict(factor=6.0, original=2048, fast=16.0, slow=2.0)),
                           (16, 10000.0, None), (6, 100.0, dict(factor=2.0, original=4096, fast=1.0, slow=1.0)),
                           (4, 10.0, dict(factor=3.0, original=100000, fast=0.001, slow=0.0001)), (32, 1000.0, dict(factor=0.5, original=8, fast=64.0, slow=32.0))):
        f, mag = scaled_pair_inv_freq(base, dims, sc)
        fw, mw = ref.scaled_frequencies(dims, base, sc)
        assert f.dtype == torch.float32 and f.numel() == dims // 2
        assert float(((f.double() - fw).abs() / fw).max()) < 1e-7 and abs(mag - mw) < 1e-12, (dims, base, sc)


def check_scaled_rotation(ops, device, dtype, T=9, H=3, d=20, rot_dims=12, eps=1e-5):
    """Head norm, rotation of the first rot_dims features in the half-split pairing with scaled frequencies and a magnitude
    on cos and sin; far positions; into a new tensor and into cache rows."""
    g = torch.Generator().manual_seed(4)
    sc = dict(factor=4.0, original=64, fast=4.0, slow=0.5)
    f, mag = ref.scaled_frequencies(rot_dims, 300.0, sc)
    assert mag != 1.0
    src = _bf(torch.randn(T, H * d + 4, generator=g) * 2)
    w = _bf(1 + 0.1 * torch.randn(d, generator=g))
    pos = torch.tensor([0, 1, 2, 3, 500, 501, 4095, 7, 8])
    x = src[:, 1: 1 + H * d].reshape(T, H, d)
    normed = ref.unit_rms(x, eps) * w
    full = torch.zeros(4096, H, d, dtype=torch.float64)
    full[pos] = normed
    want = ref.rotate_half(full, rot_dims, f, mag)[pos]
    sd = src.to(dtype).to(device)[:, 1: 1 + H * d].view(T, H, d)
    got = ops.head_norm_rope(sd, w.to(dtype).to(device), eps, pos.to(device), f.float().to(device), rot_dims, False, 1.0, dtype, rot_mag=mag)
    _close(got, want, 3e-4 if dtype == torch.float32 else _tol(dtype), "head norm and scaled rotation")
    assert torch.equal(got[..., rot_dims:].cpu().double(), normed[..., rot_dims:].to(dtype).double()) or dtype == torch.float32
    cache = torch.zeros(40, H, d, dtype=dtype, device=device)
    loc = torch.tensor([3, 9, 1, 30, 12, 2, 5, 39, 17], device=device)
    ops.head_norm_rope(sd, w.to(dtype).to(device), eps, pos.to(device), f.float().to(device), rot_dims, False, 1.0, dtype, cache=cache, loc=loc,
                       rot_mag=mag)
    _close(cache[loc], want, 3e-4 if dtype == torch.float32 else _tol(dtype), "the same into cache rows")
    assert float(cache[0].abs().max()) == 0.0 and float(cache[4].abs().max()) == 0.0
    # the values' norm: a unit weight, no rotation
    ones = torch.ones(d, dtype=dtype, device=device)
    got = ops.head_norm_rope(sd, ones, eps, pos.to(device), f.float().to(device), 0, False, 1.0, dtype)
    _close(got, ref.unit_rms(x, eps), _tol(dtype), "division by the root mean square alone")


def check_qkv_norms_one_launch(ops, device, dtype, T=11, H=5, G=2, d=20, dv=12, rot_dims=8, eps=1e-5):
    """q, k and v of a stacked projection through the one launch: against the oracle, and equal to the three single launches."""
    g = torch.Generator().manual_seed(9)
    f, mag = ref.scaled_frequencies(rot_dims, 300.0, dict(factor=4.0, original=64, fast=4.0, slow=0.5)) if rot_dims else (torch.zeros(0), 1.0)
    width = (H + G) * d + G * dv
    src = _bf(torch.randn(T, width + 3, generator=g) * 2)
    wq, wk = (_bf(1 + 0.1 * torch.randn(d, generator=g)) for _ in range(2))
    pos = torch.arange(T) + 700
    sd = src.to(dtype).to(device)
    q, k, v = sd[:, : H * d].view(T, H, d), sd[:, H * d: (H + G) * d].view(T, G, d), sd[:, (H + G) * d: width].view(T, G, dv)
    loc = (torch.randperm(30, generator=g)[:T] + 1).to(device)
    kc, vc = torch.zeros(32, G, d, dtype=dtype, device=device), torch.zeros(32, G, dv, dtype=dtype, device=device)
    fd = f.float().to(device)
    got = ops.qkv_norm_rope_write(q, k, v, wq.to(dtype).to(device), wk.to(dtype).to(device), eps, pos.to(device), fd, rot_dims, False, mag, kc, vc, loc)
    full = torch.zeros(T + 700, H + G, d, dtype=torch.float64)
    x = src[:, : (H + G) * d].reshape(T, H + G, d)
    full[pos] = torch.cat([ref.unit_rms(x[:, :H], eps) * wq, ref.unit_rms(x[:, H:], eps) * wk], 1)
    want = ref.rotate_half(full, rot_dims, f, mag)[pos] if rot_dims else full[pos]
    tol = 3e-4 if dtype == torch.float32 else _tol(dtype)
    _close(got, want[:, :H], tol, "queries of the one launch")
    _close(kc[loc], want[:, H:], tol, "keys of the one launch, in their cache rows")
    _close(vc[loc], ref.unit_rms(src[:, (H + G) * d: width].reshape(T, G, dv), eps), tol, "values of the one launch, in their cache rows")
    assert float(kc[0].abs().max()) == 0.0 and float(vc[0].abs().max()) == 0.0
    q1 = ops.head_norm_rope(q, wq.to(dtype).to(device), eps, pos.to(device), fd, rot_dims, False, 1.0, dtype, rot_mag=mag)
    k1 = torch.zeros_like(kc)
    ops.head_norm_rope(k, wk.to(dtype).to(device), eps, pos.to(device), fd, rot_dims, False, 1.0, dtype, cache=k1, loc=loc, rot_mag=mag)
    assert torch.equal(got, q1) and torch.equal(kc, k1), "the one launch and the single launches round alike"


# ------------------------------------------------------------------------------------------- convolution with bias
def run_conv(ops, device, dtype, u, w, bias, cuts, act, slot=2, decode_tail=0):
    T, C = u.shape
    taps = w.shape[1]
    tab = Table(device)
    tab.req_to_state[4] = slot
    state = torch.full((5, taps - 1, C), 55.0, dtype=torch.float32, device=device)      # stale: position 0 must not read it
    wide = torch.zeros(T, C + 8, dtype=dtype)
    wide[:, 8:] = u.to(dtype)
    ud = wide.to(device)[:, 8:]
    outs, at = [], 0
    for n in cuts:
        decode = at >= T - decode_tail and n == 1
        b = tab.batch([(4, at, n)])
        y = ops.causal_conv(ud[at:at + n], w.to(dtype).to(device), state, tab.req_to_state, b["req_pool_indices"], b["positions"],
                            act=act, bias=None if bias is None else bias.to(dtype).to(device), **_segs(b, decode))
        outs.append(y.cpu())
        at += n
    assert at == T
    return torch.cat(outs)


def check_conv_bias(ops, device, dtype, C=40, T=33):
    g = torch.Generator().manual_seed(6)
    for taps, cuts, tail in ((4, (T,), 0), (4, (5, 2, 1, T - 13, 1, 1, 1, 2), 0), (3, (T - 3, 1, 1, 1), 3), (2, (1,) * T, T), (1, (T,), 0)):
        u = _bf(torch.randn(T, C, generator=g))
        w = _bf(torch.randn(C, taps, generator=g) * 0.6)
        b = _bf(torch.randn(C, generator=g))
        want = ref.silu(ref.causal_conv(u, w, b))
        got = run_conv(ops, device, dtype, u, w, b, cuts, "silu", decode_tail=tail)
        _close(got, want, _tol(dtype), f"convolution of {taps} taps with bias and silu, cut into {list(cuts)[:6]}")
    # 37 channels: no whole 16-byte groups
    u, w, b = _bf(torch.randn(T, 37, generator=g)), _bf(torch.randn(37, 4, generator=g)), _bf(torch.randn(37, generator=g))
    _close(run_conv(ops, device, dtype, u, w, b, (7, 2, T - 9), "none"), ref.causal_conv(u, w, b), _tol(dtype), "odd channel count")


# ------------------------------------------------------------------------------------------- state-space recurrence
def run_state_space(ops, device, dtype, x, B, C, dt_logits, dt_bias, rate_log, skip, cuts, slot=2, decode_tail=0, state=None, qk_fp32=False):
    T, H, dv = x.shape
    G, N = B.shape[1], B.shape[2]
    tab = Table(device)
    tab.req_to_state[4] = slot
    if state is None:
        state = torch.full((5, H, N, dv), 77.0, dtype=torch.float32, device=device)     # stale: position 0 must not read it
    qt = torch.float32 if qk_fp32 else dtype
    wide = torch.zeros(T, H * dv + 2 * G * N, dtype=dtype)
    wide[:, : H * dv] = x.reshape(T, -1).to(dtype)
    wide[:, H * dv: H * dv + G * N] = B.reshape(T, -1).to(dtype)
    wide[:, H * dv + G * N:] = C.reshape(T, -1).to(dtype)
    wd = wide.to(device)
    xd = wd[:, : H * dv].view(T, H, dv)
    Bd = wd[:, H * dv: H * dv + G * N].view(T, G, N).to(qt)
    Cd = wd[:, H * dv + G * N:].view(T, G, N).to(qt)
    zd = dt_logits.float().to(device)
    outs, at = [], 0
    for n in cuts:
        decode = at >= T - decode_tail and n == 1
        b = tab.batch([(4, at, n)])
        o = torch.empty((n, H, dv), dtype=torch.float32, device=device)
        ops.linear_recurrence(Cd[at:at + n], Bd[at:at + n], xd[at:at + n], o, state, tab.req_to_state, b["req_pool_indices"],
                              b["positions"], 1.0, dt_logits=zd[at:at + n], dt_bias=dt_bias.float().to(device),
                              rate_log=rate_log.float().to(device), skip=None if skip is None else skip.float().to(device),
                              **_segs(b, decode))
        outs.append(o.cpu())
        at += n
    assert at == T
    return torch.cat(outs), state


def check_state_space(ops, device, dtype, H=4, G=2, N=10, dv=20, T=45, cuts=(45,), decode_tail=0, with_skip=True):
    g = torch.Generator().manual_seed(2)
    x = _bf(torch.randn(T, H, dv, generator=g))
    B = _bf(torch.randn(T, G, N, generator=g) * 0.5)
    C = _bf(torch.randn(T, G, N, generator=g) * 0.5)
    z = torch.randn(T, H, generator=g).float().double()
    dt_bias = _bf(torch.randn(H, generator=g) - 1.0)
    rate_log = _bf(torch.randn(H, generator=g) * 0.5)
    skip = _bf(1 + 0.3 * torch.randn(H, generator=g)) if with_skip else None
    want = ref.state_space_recurrence(x, B, C, ref.softplus(z + dt_bias), torch.exp(rate_log), skip)
    got, _ = run_state_space(ops, device, dtype, x, B, C, z, dt_bias, rate_log, skip, cuts, decode_tail=decode_tail)
    _close(got, want, 5e-5, f"state-space recurrence ({H} heads in {G} groups, state {N}, width {dv}) cut into {list(cuts)[:6]}")


def check_state_space_planted(ops, device, dtype):
    """A write 500 tokens back under a key that nothing else uses is read in full by a head that does not decay, and is
    gone from a head that does; a large step-size logit passes through softplus unclamped; a stale slot is not read at
    position 0 but IS read by a continued sequence."""
    H, G, N, dv, T = 2, 1, 8, 4, 520
    x = torch.zeros(T, H, dv, dtype=torch.float64)
    B = torch.zeros(T, G, N, dtype=torch.float64)
    C = torch.zeros(T, G, N, dtype=torch.float64)
    z = torch.zeros(T, H, dtype=torch.float64)
    B[:, 0, 1] = 1.0                      # every token writes under key 1
    B[3, 0] = 0
    B[3, 0, 0] = 1.0                      # token 3 alone writes under key 0
    x[3, :, 2] = 2.0
    C[T - 1, 0, 0] = 1.0                  # the last token reads key 0
    z[3] = 30.0                           # a step of 30 (softplus is the identity there, nothing clamps it)
    dt_bias = torch.zeros(H)
    rate_log = torch.tensor([-40.0, -3.0])          # head 0 keeps everything, head 1 forgets at exp(-3) per unit step
    for cuts, tail in (([T], 0), ([2, 2, 400, 1, 1, T - 406], 0), ([T - 2, 1, 1], 2)):
        got, state = run_state_space(ops, device, dtype, x, B, C, z, dt_bias, rate_log, None, cuts, decode_tail=tail)
        assert abs(float(got[T - 1, 0, 2]) - 60.0) < 1e-3, cuts                  # dt * B x = 30 * 2, kept over 516 tokens
        steps = (T - 4) * math.log(2.0)                                          # softplus(0) per later token
        assert abs(float(got[T - 1, 1, 2]) - 60.0 * math.exp(-math.exp(-3.0) * steps)) < 1e-3, cuts
        assert float(got[:T - 1].abs().max()) == 0.0
    # the slot's matrix afterwards is what a continuation reads: one more token that reads key 0 sees the same value
    b = Table(device)
    b.req_to_state[4] = 2
    bb = b.batch([(4, T, 1)])
    o = torch.empty((1, H, dv), dtype=torch.float32, device=device)
    q1 = torch.zeros(1, G, N, dtype=torch.float32, device=device)
    q1[0, 0, 0] = 1.0
    zeros = torch.zeros(1, G, N, dtype=torch.float32, device=device)
    ops.linear_recurrence(q1, zeros, torch.zeros(1, H, dv, dtype=dtype, device=device), o, state, b.req_to_state, bb["req_pool_indices"],
                          bb["positions"], 1.0, dt_logits=torch.full((1, H), -50.0, device=device), dt_bias=dt_bias.to(device),
                          rate_log=rate_log.to(device), skip=None)
    assert abs(float(o[0, 0, 2]) - 60.0) < 1e-3


# ------------------------------------------------------------------------------------------- delta rule, one decay per head
def run_delta_rule(ops, device, dtype, q, k, v, beta_logits, z, rate_bias, rate_log, cuts, q_scale=1.0, slot=2, decode_tail=0, state=None):
    T, G, dk = q.shape
    H, dv = v.shape[1], v.shape[2]
    tab = Table(device)
    tab.req_to_state[4] = slot
    if state is None:
        state = torch.full((5, H, dk, dv), 77.0, dtype=torch.float32, device=device)
    qd, kd = q.float().to(device), k.float().to(device)
    vd = v.to(dtype).to(device)
    ba = torch.cat([beta_logits, z], 1).float().to(device)          # [beta | decay logits] side by side, fp32
    outs, at = [], 0
    for n in cuts:
        decode = at >= T - decode_tail and n == 1
        b = tab.batch([(4, at, n)])
        o = torch.empty((n, H, dv), dtype=torch.float32, device=device)
        ops.gated_delta_rule(qd[at:at + n], kd[at:at + n], vd[at:at + n], ba[at:at + n, :H], ba[at:at + n, H:], rate_bias.float().to(device),
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
    beta_logits = torch.randn(T, H, generator=g).float().double()
    z = torch.randn(T, H, generator=g).float().double()
    rate_bias = _bf(torch.randn(H, generator=g) - 1.0)
    rate_log = _bf(torch.randn(H, generator=g) * 0.5)
    decay = torch.exp(-torch.exp(rate_log) * ref.softplus(z + rate_bias))
    want = ref.gated_delta_rule(q * 0.37, k, v, torch.sigmoid(beta_logits), decay)
    got, _ = run_delta_rule(ops, device, dtype, q, k, v, beta_logits, z, rate_bias, rate_log, cuts, q_scale=0.37, decode_tail=decode_tail)
    _close(got, want, 5e-5, f"delta rule with a decay per head ({H}/{G} heads of {dk}/{dv}) cut into {list(cuts)[:6]}")


def check_delta_rule_planted(ops, device, dtype):
    """A value written 600 tokens back under its own key is read in full by a head that does not decay, REPLACED by a second
    write under the same key (beta 1), and forgotten by a head that decays; a token's read-out already holds what the token itself wrote."""
    H, G, dk, dv, T = 2, 1, 8, 4, 620
    q = torch.zeros(T, G, dk, dtype=torch.float64)
    k = torch.zeros(T, G, dk, dtype=torch.float64)
    v = torch.zeros(T, H, dv, dtype=torch.float64)
    k[:, 0, 1] = 1.0
    k[5, 0] = 0
    k[5, 0, 0] = 1.0
    v[5, :, 3] = 7.0
    k[610, 0] = 0
    k[610, 0, 0] = 1.0
    v[610, :, 3] = -2.0
    for t in (5, 609, 610, T - 1):
        q[t, 0, 0] = 1.0
    beta = torch.full((T, H), 40.0, dtype=torch.float64)           # sigmoid = 1
    z = torch.zeros(T, H, dtype=torch.float64)
    rate_bias = torch.zeros(H)
    rate_log = torch.tensor([-40.0, -4.0])
    for cuts, tail in (([T], 0), ([5, 1, 300, 2, 301, 1, 10], 0), ([T - 11] + [1] * 11, 11)):
        got, _ = run_delta_rule(ops, device, dtype, q, k, v, beta, z, rate_bias, rate_log, cuts, decode_tail=tail)
        assert abs(float(got[5, 0, 3]) - 7.0) < 1e-4, cuts                       # its own write, read in the same step
        assert abs(float(got[609, 0, 3]) - 7.0) < 1e-3, cuts                     # 604 tokens later, nothing lost
        assert abs(float(got[610, 0, 3]) + 2.0) < 1e-3 and abs(float(got[T - 1, 0, 3]) + 2.0) < 1e-3, cuts       # replaced, not added
        keep = math.exp(-math.exp(-4.0) * math.log(2.0) * 604)
        assert abs(float(got[609, 1, 3]) - 7.0 * keep) < 1e-3, cuts


# ------------------------------------------------------------------------------------------- window attention with averaged blocks
def run_pooled_attention(ops, device, dtype, q, kn, v, scale, window, pool, cuts, page=1, decode_tail=0, sink=None, gate=None, splits=1,
                         stale=False):
    """The keys and values are in the cache rows beforehand; every step first writes the averages of the blocks it completes
    (as the layer does after its cache write), then attends.  sink [H] or None; gate [T, H] logits or None."""
    T, H, d = q.shape
    G, dv = kn.shape[1], v.shape[-1]
    kv = KVSetup(device, dtype, kn, v, page=page)
    div = pool if (pool > 0 and page % pool == 0) else 1
    rows = (kv.k_cache.shape[0] + div - 1) // div
    fill = 9.0 if stale else 0.0            # stale averages: a block's row is written before anything reads it
    pk = torch.full((rows, G, d), fill, dtype=dtype, device=device)
    pv = torch.full((rows, G, dv), fill, dtype=dtype, device=device)
    bq = ops.window_attention_block_tokens(H, G, d, dv, dtype)
    qd = q.to(dtype).to(device)
    gd = None
    if gate is not None:
        wide = torch.zeros(T, H + 3, dtype=dtype)
        wide[:, 1: 1 + H] = gate.to(dtype)
        gd = wide.to(device)[:, 1: 1 + H]
    sk = None if sink is None else sink.float().to(device)
    outs, at = [], 0
    for n in cuts:
        decode = at >= T - decode_tail and n == 1
        b = kv.tab.batch([(kv.row, at, n)])
        tr = None if decode else b["tok_req"]
        if pool > 0:
            ops.pool_kv_blocks(kv.k_cache, kv.v_cache, pk, pv, kv.tab.req_to_token, b["req_pool_indices"], b["positions"], pool, div, tok_req=tr)
        o = torch.zeros((n, H, dv), dtype=dtype, device=device)
        blocks = None
        if not decode:
            blocks = torch.tensor([[s, min(bq, n - s)] for s in range(0, n, bq)], dtype=torch.int32, device=device)
        ops.window_attention(qd[at:at + n], kv.k_cache, kv.v_cache, o, kv.tab.req_to_token, b["req_pool_indices"], b["positions"], sk,
                             window, scale, tok_req=tr, blocks=blocks, max_run=bq, num_splits=splits if decode else 1, pool=pool,
                             pooled_k=pk if pool > 0 else None, pooled_v=pv if pool > 0 else None, pool_div=div,
                             head_gate=None if gd is None else gd[at:at + n])
        outs.append(o.cpu())
        at += n
    assert at == T
    return torch.cat(outs)


def check_pooled_attention(ops, device, dtype, H=4, G=2, d=32, dv=32, T=150, window=40, pool=8, cuts=(150,), page=1, decode_tail=0,
                           splits=1, with_gate=True):
    g = torch.Generator().manual_seed(3)
    q = _bf(torch.randn(T, H, d, generator=g))
    kn = _bf(torch.randn(T, G, d, generator=g))
    v = _bf(torch.randn(T, G, dv, generator=g))
    sink = _bf(torch.randn(H, generator=g))
    gate = _bf(torch.randn(T, H, generator=g) * 2) if with_gate else None
    scale = 1.7 / math.sqrt(d)
    want = ref.pooled_window_attention(q, kn, v, scale, window, pool, sink)
    if gate is not None:
        want = want * torch.sigmoid(gate)[:, :, None]
    got = run_pooled_attention(ops, device, dtype, q, kn, v, scale, window, pool, cuts, page=page, decode_tail=decode_tail, sink=sink,
                               gate=gate, splits=splits, stale=True)
    _close(got, want, 2e-5 if dtype == torch.float32 else 1.5e-2,
           f"attention over a window of {window} and blocks of {pool} ({H}/{G} heads of {d}/{dv}) cut into {list(cuts)[:6]}, pages of {page}")


def check_pooled_attention_planted(ops, device, dtype, d=32, W=24, P=8, page=1):
    """Scores are zero except where a query meets a planted key (score 16).  A key inside a block is seen through the block's
    average (a P-th of its score and of its value) exactly from the token at which the whole block lies before the window,
    b P + P - 1 <= i - W; between leaving the window and that token nothing shows it; the first block and a far block
    among many stay visible to the end; in prompts, portions and decode steps alike."""
    H, G, T = 2, 1, 40 * P + 5
    assert P >= 3
    jb = 5 * P + 1                               # a key in block 5, not its last: P - 2 tokens see neither it nor its block
    q = torch.zeros(T, H, d, dtype=torch.float64)
    kn = torch.zeros(T, G, d, dtype=torch.float64)
    v = torch.zeros(T, G, d, dtype=torch.float64)
    kn[jb, 0, 1] = 4.0 * P                       # its block's average holds 4.0 in column 1
    v[jb, 0, 1] = 1.0 * P                        # ... and 1.0 as value
    kn[1, 0, 2] = 4.0 * P                        # a key in the very first block
    v[1, 0, 2] = 3.0 * P
    last_in = jb + W - 1                         # the last token whose window holds jb itself
    first_pooled = 5 * P + P - 1 + W             # the first token that sees block 5
    asks = [last_in, last_in + 1, first_pooled - 1, first_pooled, T - 1]
    for i in asks:
        q[i, :, 1] = 4.0
    q[T - 1, :, 2] = 4.0
    hot = math.exp(16.0)
    tol = 1e-5 if dtype == torch.float32 else 1e-2

    def blocks_seen(i):
        return max(0, (i - W + 1) // P)

    def cut_at(points):
        edges = sorted(set(p for p in points if 0 < p < T)) + [T]
        return [b - a for a, b in zip([0] + edges[:-1], edges)]

    for cuts, tail in (([T], 0), (cut_at([last_in, last_in + 1, last_in + 2, first_pooled - 1, first_pooled, first_pooled + 1]), 0),
                       (cut_at([first_pooled - 2, first_pooled - 1, first_pooled, first_pooled + 1, first_pooled + 2]), 0), ([T - 1, 1], 1),
                       (cut_at([first_pooled]), 0)):
        assert sum(cuts) == T
        for splits in ((1, 3) if tail else (1,)):
            got = run_pooled_attention(ops, device, dtype, q, kn, v, 1.0, W, P, cuts, page=page, decode_tail=tail, splits=splits, stale=True).double()
            # the key itself, in the window: score 4 * 4 P would overflow nothing in fp32 only for small P, so compare by ratio
            s_in = math.exp(min(16.0 * P, 80.0))
            i = last_in
            den = s_in + (W - 1) + blocks_seen(i)
            assert abs(float(got[i, 0, 1]) - P * s_in / den) < tol * P, (cuts, "in the window")
            for i in (last_in + 1, first_pooled - 1):      # out of the window, its block not complete before the window yet
                assert abs(float(got[i, 0, 1])) < 1e-6, (cuts, i, "between window and block")
            i = first_pooled
            den = hot + W + (blocks_seen(i) - 1)
            assert abs(float(got[i, 1, 1]) - hot / den) < tol, (cuts, "the block is seen")
            i = T - 1                                      # both planted blocks among 30-odd, far back
            den = 2 * hot + W + (blocks_seen(i) - 2)
            assert abs(float(got[i, 0, 1]) - hot / den) < tol and abs(float(got[i, 1, 2]) - 3.0 * hot / den) < tol, (cuts, "far blocks")
            assert float(got[0].abs().max()) == 0.0
    # the same edges passed token by token in decode steps (one launch per token, key ranges merged by a second launch)
    Tt = first_pooled + 2
    n1 = Tt - last_in + 1
    for splits in (1, 2):
        got = run_pooled_attention(ops, device, dtype, q[:Tt], kn[:Tt], v[:Tt], 1.0, W, P, [last_in - 1] + [1] * n1, page=page, decode_tail=n1,
                                   splits=splits, stale=True).double()
        assert abs(float(got[last_in, 0, 1]) - P) < tol * P, "decoded: in the window"
        assert abs(float(got[last_in + 1, 0, 1])) < 1e-6 and abs(float(got[first_pooled - 1, 1, 1])) < 1e-6, "decoded: between window and block"
        den = hot + W + (blocks_seen(first_pooled) - 1)
        assert abs(float(got[first_pooled, 1, 1]) - hot / den) < tol, "decoded: the block is seen"
