"""CPU checker implementation of the ops surface the host-side layers call (tests only).

Installed with sglang_custom_amd.ops_backend.set_ops_backend() so that the batch plumbing, the
model wiring and tensor-parallel sharding can be exercised without a GPU; every function is the
oracle's restatement of the reference op, adapted to the calling convention of
sglang_custom_amd.ops (pre-allocated / in-place outputs)."""
import torch
import torch.nn.functional as F

from oracle import ops_ref


def rmsnorm(x, weight, eps, out=None):
    y = ops_ref.rmsnorm(x, weight, eps)
    if out is None:
        return y
    out.copy_(y)
    return out


def fused_add_rmsnorm(x, residual, weight, eps):
    y, r = ops_ref.rmsnorm(x, weight, eps, residual)
    x.copy_(y)
    residual.copy_(r)


def silu_and_mul(x, out=None):
    y = ops_ref.silu_and_mul(x)
    if out is None:
        return y
    out.copy_(y)
    return out


def softcap_inplace(logits, cap):
    logits.copy_(ops_ref.softcap(logits, cap))
    return logits


def rope_inplace(positions, q, k, head_size, cos_sin_cache, is_neox, v=None, k_buffer=None,
                 v_buffer=None, loc=None):
    qn, kn = ops_ref.apply_rope(positions, q, k, head_size, cos_sin_cache, is_neox)
    q.copy_(qn)
    k.copy_(kn)
    if k_buffer is not None:
        T = positions.numel()
        k_buffer[loc.long()] = k.reshape(T, -1, head_size)
        v_buffer[loc.long()] = v.reshape(T, -1, v_buffer.shape[-1])


def set_kv_buffer(k_buffer, v_buffer, loc, cache_k, cache_v):
    T = loc.numel()
    k_buffer[loc.long()] = cache_k.reshape(T, *k_buffer.shape[1:])
    v_buffer[loc.long()] = cache_v.reshape(T, *v_buffer.shape[1:])


def embedding(ids, table, vocab_start=0, vocab_end=None):
    if vocab_end is None:
        vocab_end = vocab_start + table.shape[0]
    ok = (ids >= vocab_start) & (ids < vocab_end)
    out = table[(ids - vocab_start).clamp(0, table.shape[0] - 1)]
    out = out * ok.unsqueeze(-1).to(out.dtype)
    return out


def create_kv_indices(req_to_token, req_pool_indices, page_kernel_lens, kv_indptr, kv_start_idx, kv_indices):
    r = ops_ref.create_kv_indices(req_to_token, req_pool_indices, page_kernel_lens, kv_start_idx)
    kv_indices[: r.numel()] = r


def write_req_to_token(req_to_token, req_pool_indices, pre_lens, seq_lens, extend_lens, out_cache_loc):
    ops_ref.write_req_to_token(req_to_token, req_pool_indices, pre_lens, seq_lens, out_cache_loc)


def compute_position(extend_prefix_lens, extend_seq_lens, extend_seq_lens_sum):
    pos, start = ops_ref.compute_position(extend_prefix_lens, extend_seq_lens)
    return pos, start.to(torch.int32)


def prepare_decode(req_to_token, req_pool_indices, seq_lens, out_cache_loc, positions):
    seq_lens.add_(1)
    positions.copy_(ops_ref.clamp_position(seq_lens))
    req_to_token[req_pool_indices, seq_lens - 1] = out_cache_loc.to(torch.int32)


def decode_num_splits(bs, hkv, max_seq_len, max_splits):
    return 1


def decode_attention_paged(q, k_buffer, v_buffer, o, req_to_token, req_pool_indices, seq_lens,
                           attn_logits, attn_lse, num_kv_splits, sm_scale, logit_cap=0.0, tickets=None, kv_chunk_keys=None):
    assert logit_cap == 0.0
    gqa = q.shape[1] != k_buffer.shape[1]
    o.copy_(ops_ref.decode_attention(q, k_buffer, v_buffer, req_to_token, req_pool_indices, seq_lens,
                                     sm_scale, gqa))


def decode_attention_mla(q, kv_buffer, o, req_to_token, req_pool_indices, seq_lens, attn_logits, attn_lse,
                         num_kv_splits, kv_lora_rank, sm_scale, logit_cap=0.0, tickets=None, kv_chunk_keys=None):
    """Multi-query attention over latent rows: keys = whole rows, values = their first kv_lora_rank features."""
    assert not logit_cap
    o.copy_(ops_ref.decode_attention(q, kv_buffer, kv_buffer[..., :kv_lora_rank], req_to_token, req_pool_indices,
                                     seq_lens, sm_scale, True))


def extend_attention_fwd(q_extend, k_extend, v_extend, o_extend, k_buffer, v_buffer, qo_indptr,
                         kv_indptr, kv_indices, custom_mask, is_causal, mask_indptr, max_len_extend,
                         sm_scale=None, logit_cap=0.0, skip_prefix_custom_mask=True,
                         sliding_window_size=-1):
    """Prefix keys come from kv_indices, new keys from k_extend/v_extend (extend_attention.py:306-438)."""
    assert custom_mask is None and logit_cap == 0.0 and sliding_window_size in (-1, None)
    Hq, Hkv = q_extend.shape[1], k_extend.shape[1]
    for i in range(qo_indptr.numel() - 1):
        qs, qe = int(qo_indptr[i]), int(qo_indptr[i + 1])
        ps, pe = int(kv_indptr[i]), int(kv_indptr[i + 1])
        idx = kv_indices[ps:pe].long()
        if pe > ps:
            k = torch.cat([k_buffer[idx], k_extend[qs:qe]], 0).movedim(0, 1)
            v = torch.cat([v_buffer[idx], v_extend[qs:qe]], 0).movedim(0, 1)
        else:   # no prefix: the buffers are not read (an MLA pool's rows do not even have this shape)
            k, v = k_extend[qs:qe].movedim(0, 1), v_extend[qs:qe].movedim(0, 1)
        ext, pre = qe - qs, pe - ps
        qq = torch.zeros((Hq, pre + ext, q_extend.shape[2]), dtype=q_extend.dtype)
        qq[:, pre:] = q_extend[qs:qe].movedim(0, 1)
        o = F.scaled_dot_product_attention(qq[None], k[None], v[None], enable_gqa=Hq != Hkv,
                                           scale=sm_scale, is_causal=is_causal)
        o_extend[qs:qe] = o[0].movedim(1, 0)[pre:]


def linear(x, weight, bias=None, out_dtype=None):
    y = F.linear(x, weight, bias)
    return y if out_dtype is None else y.to(out_dtype)


def argmax(logits):
    return ops_ref.greedy(logits)


def softmax_temperature_(logits, temperatures):
    logits.copy_(ops_ref.softmax_temperature(logits, temperatures.view(-1, 1)))
    return logits


def top_k_top_p_min_p_sample(probs, top_ks, top_ps, min_ps, uniform):
    kept = ops_ref.kept_distribution(probs, top_ks, top_ps, min_ps)
    cdf = kept.cumsum(-1)
    return (cdf < uniform.view(-1, 1) * cdf[:, -1:]).sum(-1).clamp(max=probs.shape[1] - 1).to(torch.int32)


def alloc_extend_pages(prefix_lens, seq_lens, last_loc, free_pages, page_size, extend_num_tokens):
    out, used = ops_ref.alloc_extend_pages(prefix_lens, seq_lens, last_loc, free_pages, page_size)
    assert out.numel() == extend_num_tokens
    return out, used


def alloc_decode_pages(seq_lens, last_loc, free_pages, page_size):
    return ops_ref.alloc_decode_pages(seq_lens, last_loc, free_pages, page_size)


def qkv_proj_rope_tiled_supported(m, k, num_heads, num_kv_heads, head_dim, rotary_dim, is_neox, dtype, fp8):
    """The fused prefill projection + RoPE + cache write is a GPU kernel only: the double declines and the
    model takes the unfused sequence, which is what the oracle restates."""
    return False


def decode_attention_mla_fused_rope_supported(kv_lora_rank, rope_dim, dtype, cache_dtype):
    """RoPE + latent-row write inside the MLA decode launch is a GPU kernel only: the double declines and the
    model takes rotary_emb + set_kv_buffer + decode_attention_mla, which is what the oracle restates."""
    return False


def mla_latent_norms_supported(q_rank, kv_rank, rope_dim, dtype):
    """The one-launch q_a / kv_a norms are a GPU kernel only: the double declines and the model takes
    split + contiguous + rmsnorm, which is what the oracle restates."""
    return False


def mla_absorb_supported(m, n, k, tail, dtype):
    """The one-launch absorbed products are a GPU kernel only: the double declines and the model takes
    torch.bmm + cat / transpose, which is what the oracle restates."""
    return False


def mla_prefill_assemble_supported(nope, rope, vd, rank, dtype):
    """The one-launch prefill glue is a GPU kernel only: the double declines and the model takes rotary_emb + the
    copies + set_kv_buffer, which is what the oracle restates."""
    return False


# ------------------------------------------------------- fp32 residual stream with per-sequence state
# Restatements of what the header says of each kernel (include/mi355_hotpath.h) token by token; they share nothing with the
# whole-sequence functions of oracle/seturax_ref.py that the tests compare against.
def _segments(T, tok_req, seg_start, seg_len):
    """(b, first, last) per token."""
    if tok_req is None:
        return [(t, True, True) for t in range(T)]
    out = []
    for t in range(T):
        b = int(tok_req[t])
        s, n = int(seg_start[b]), int(seg_len[b])
        out.append((b, t == s, t == s + n - 1))
    return out


def bigram_embedding(ids, table, bigram, prev_token, req_to_state, req_pool_indices, positions, scale, mul_prev, mul_cur,
                     buckets, tok_req=None, seg_start=None, seg_len=None):
    T = ids.numel()
    x = torch.empty((T, table.shape[1]), dtype=torch.float32)
    for t, (b, first, _) in enumerate(_segments(T, tok_req, seg_start, seg_len)):
        tok = int(ids[t])
        if int(positions[t]) == 0:
            row = buckets
        else:
            prev = int(prev_token[int(req_to_state[int(req_pool_indices[b])])]) if first else int(ids[t - 1])
            row = (prev * mul_prev + tok * mul_cur) % buckets
        x[t] = table[tok].float() * scale + bigram[row].float()
    return x


def _ln(row, w, eps):
    mu = row.mean()
    var = ((row - mu) ** 2).mean()
    return (row - mu) / torch.sqrt(var + eps) * w.float()


def layernorm_shift(x, weight, eps, shift=None, state=None, req_to_state=None, req_pool_indices=None, positions=None,
                    h_last=None, tok_req=None, seg_start=None, seg_len=None):
    T, D = x.shape
    h32 = torch.stack([_ln(x[t], weight, eps) for t in range(T)]) if T else x.new_zeros((0, D))
    if shift is None:
        return h32.to(weight.dtype)
    hs = torch.empty_like(h32)
    for t, (b, first, last) in enumerate(_segments(T, tok_req, seg_start, seg_len)):
        if int(positions[t]) == 0:
            prev = torch.zeros(D)
        elif first:
            prev = state[int(req_to_state[int(req_pool_indices[b])])]
        else:
            prev = h32[t - 1]
        hs[t] = h32[t] + (prev - h32[t]) * shift.float()
        if last and h_last is not None:
            h_last[b] = h32[t]
    return h32.to(weight.dtype), hs.to(weight.dtype)


def commit_sequence_state(state, prev_token, h_last, ids, req_to_state, req_pool_indices, seg_start=None, seg_len=None):
    L, B, D = h_last.shape
    for b in range(B):
        slot = int(req_to_state[int(req_pool_indices[b])])
        state[:, slot] = h_last[:, b]
        last = b if seg_start is None else int(seg_start[b]) + int(seg_len[b]) - 1
        if prev_token is not None:
            prev_token[slot] = int(ids[last])


def gelu_tanh_and_mul(gate, up):
    z = gate.float()
    g = 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z * z * z)))
    return (g * up.float()).to(gate.dtype)


def gated_residual_add(x, g1, b1, y1, g2=None, b2=None, y2=None):
    add = torch.sigmoid(g1.float() + b1.float()) * y1.float()
    if y2 is not None:
        add = add + torch.sigmoid(g2.float() + b2.float()) * y2.float()
    x.add_(add)


def _rot(v, pos, inv_freq, rot_dims):
    half = rot_dims // 2
    ang = float(pos) * inv_freq[:half].float()
    c, s = torch.cos(ang), torch.sin(ang)
    u, w = v[..., :half].float(), v[..., half:rot_dims].float()
    return torch.cat([u * c - w * s, w * c + u * s, v[..., rot_dims:].float()], -1)


def latent_norms_rope_write(a, q_weight, kv_weight, positions, out_cache_loc, inv_freq, cache, q_rank, rank, rope_dim,
                            rot_dims, eps):
    T = a.shape[0]
    cq = torch.empty((T, q_rank), dtype=a.dtype)
    for t in range(T):
        row = a[t].float()
        q = row[:q_rank]
        cq[t] = (q / torch.sqrt((q * q).mean() + eps) * q_weight.float()).to(a.dtype)
        c = row[q_rank: q_rank + rank]
        c = c / torch.sqrt((c * c).mean() + eps) * kv_weight.float()
        kr = _rot(row[q_rank + rank: q_rank + rank + rope_dim], positions[t], inv_freq, rot_dims)
        cache[int(out_cache_loc[t])] = torch.cat([c, kr]).to(cache.dtype)
    return cq


def latent_window_attention_block_tokens(heads, rank, rope_dim, dtype):
    return 3


def latent_window_attention_splits(tokens, heads, rank, window, max_position, dtype):
    return 1


def latent_window_attention(qa, qr, cache, out, req_to_token, req_pool_indices, positions, sink, inv_freq, rot_dims, window,
                            scale, gate=None, tok_req=None, blocks=None, num_splits=1):
    T, H, rank = qa.shape
    covered = torch.zeros(T, dtype=torch.bool)
    runs = [(t, 1) for t in range(T)] if blocks is None else [(int(a), int(n)) for a, n in blocks.tolist()]
    for t0, n in runs:
        for t in range(t0, t0 + n):
            assert not covered[t]
            covered[t] = True
            b = t if tok_req is None else int(tok_req[t])
            assert blocks is None or int(tok_req[t0]) == b, "a run crosses two sequences"
            p = int(positions[t])
            lo = max(0, p - window + 1)
            slots = req_to_token[int(req_pool_indices[b]), lo: p + 1].long()
            rows = cache[slots].float()                                  # [n_keys, rank + rope]
            q = torch.cat([qa[t].float(), _rot(qr[t], p, inv_freq, rot_dims)], -1)   # [H, rank + rope]
            s = (q @ rows.T) * scale                                     # [H, n_keys]
            m = torch.maximum(s.max(-1).values, sink.float())
            e = torch.exp(s - m[:, None])
            pr = e / (e.sum(-1) + torch.exp(sink.float() - m))[:, None]
            o = pr @ rows[:, :rank]
            if gate is not None:
                o = o * torch.sigmoid(gate[t].float())[:, None]
            out[t] = o.to(out.dtype)
    assert bool(covered.all()), "the runs do not cover every token"
    return out


# ------------------------------------------------------- post-norm stream, linear recurrences, sigmoid attention, mixture
# Token-by-token restatements of what the header says of each kernel; they share nothing with the whole-sequence
# functions of oracle/verozen_ref.py that the tests compare against.
from types import SimpleNamespace


def scaled_add_group_rmsnorm(x, branch, alpha, weight, groups, eps, rows=None, coef=None, inplace=True):
    T, D = x.shape
    s = alpha * x
    if branch is not None:
        if rows is None:
            s = s + branch.float()
        else:
            for t in range(T):
                for j in range(rows.shape[1]):
                    s[t] += float(coef[t, j]) * branch[int(rows[t, j])].float()
    part = s.view(T, groups, D // groups)
    n = (part / torch.sqrt((part * part).mean(-1, keepdim=True) + eps)).reshape(T, D) * weight.float()
    if inplace:
        x.copy_(n)
        return x if weight.dtype == torch.float32 else n.to(weight.dtype)
    return n.to(weight.dtype)


def rmsnorm_residual_add(x, y, weight, eps, offset=0.0, layer_scale=None, mult=1.0):
    y = y.float()
    n = y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps) * (offset + weight.float())
    if layer_scale is not None:
        n = n * layer_scale.float()
    x.add_(mult * n)
    return x if weight.dtype == torch.float32 else x.to(weight.dtype)


def gated_group_rmsnorm(y, gate, weight, groups, eps):
    T, D = y.shape
    g = gate.float()
    v = (y * (g * torch.sigmoid(g))).view(T, groups, D // groups)
    n = v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)
    return (n.reshape(T, D) * weight.float()).to(weight.dtype)


def head_norm_rope(src, weight, eps, positions, inv_freq, rot_dims, interleaved, scale, out_dtype, cache=None, loc=None, rot_mag=1.0):
    T, H, d = src.shape
    out = torch.empty((T, H, d), dtype=torch.float32)
    for t in range(T):
        v = src[t].float()
        if weight is not None:
            v = v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * weight.float()
        if rot_dims:
            ang = float(positions[t]) * inv_freq[: rot_dims // 2].float()
            c, s = torch.cos(ang) * rot_mag, torch.sin(ang) * rot_mag
            r = v.clone()
            if interleaved:
                a, b = v[:, 0:rot_dims:2], v[:, 1:rot_dims:2]
                r[:, 0:rot_dims:2], r[:, 1:rot_dims:2] = a * c - b * s, b * c + a * s
            else:
                a, b = v[:, : rot_dims // 2], v[:, rot_dims // 2: rot_dims]
                r[:, : rot_dims // 2], r[:, rot_dims // 2: rot_dims] = a * c - b * s, b * c + a * s
            v = r
        out[t] = v * scale
    if cache is not None:
        cache[loc.long()] = out.to(cache.dtype)
        return cache
    return out.to(out_dtype)


def qkv_norm_rope_write(q, k, v, wq, wk, eps, positions, inv_freq, rot_dims, interleaved, rot_mag, k_cache, v_cache, loc):
    head_norm_rope(k, wk, eps, positions, inv_freq, rot_dims, interleaved, 1.0, k.dtype, cache=k_cache, loc=loc, rot_mag=rot_mag)
    head_norm_rope(v, torch.ones(v.shape[2], dtype=v.dtype), eps, positions, inv_freq, 0, interleaved, 1.0, v.dtype, cache=v_cache, loc=loc)
    return head_norm_rope(q, wq, eps, positions, inv_freq, rot_dims, interleaved, 1.0, q.dtype, rot_mag=rot_mag)


def linear_recurrence(q, k, v, out, state, req_to_state, req_pool_indices, positions, q_scale, gate_logits=None, gate_bias=None,
                      tau=1.0, head_decay=None, tok_req=None, seg_start=None, seg_len=None, dt_logits=None, dt_bias=None,
                      rate_log=None, skip=None):
    T, G, dk = q.shape
    H = v.shape[1]
    rep = H // G
    S = None
    for t, (b, first, last) in enumerate(_segments(T, tok_req, seg_start, seg_len)):
        slot = int(req_to_state[int(req_pool_indices[b])])
        if first:
            S = torch.zeros_like(state[slot]) if int(positions[t]) == 0 else state[slot].clone()
        kk = k[t].float().repeat_interleave(rep, 0)
        if dt_logits is not None:
            dt = torch.nn.functional.softplus(dt_logits[t].float() + dt_bias.float())
            a = torch.exp(-torch.exp(rate_log.float()) * dt)[:, None].expand(H, dk)
            kk = kk * dt[:, None]
        elif gate_logits is not None:
            z = gate_logits[t].float() + (gate_bias.float() if gate_bias is not None else 0.0)
            a = torch.exp(torch.nn.functional.logsigmoid(z) / tau).view(H, dk)
        else:
            a = head_decay.float()[:, None].expand(H, dk)
        S = a[:, :, None] * S + kk[:, :, None] * v[t].float()[:, None, :]
        out[t] = torch.einsum("hkv,hk->hv", S, q[t].float().repeat_interleave(rep, 0) * q_scale)
        if skip is not None:
            out[t] += skip.float()[:, None] * v[t].float()
        if last:
            state[slot] = S
    return out


def head_rmsnorm_gate(o, weight, gate, eps, out_dtype):
    T, H, dv = o.shape
    n = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps)
    if weight is not None:
        n = n * weight.float()
    g = gate.float().reshape(T, H, dv)
    return (n * g * torch.sigmoid(g)).reshape(T, H * dv).to(out_dtype)


def sigmoid_attention_block_tokens(heads, kv_heads, head_dim, v_head_dim, dtype):
    return 3


def sigmoid_attention_splits(tokens, heads, kv_heads, max_len, dtype):
    return 1


def sigmoid_attention(q, k_cache, v_cache, out, req_to_token, req_pool_indices, positions, temp, bias, scale, tok_req=None,
                      blocks=None, num_splits=1, max_run=None):
    T, H, d = q.shape
    G = k_cache.shape[1]
    covered = torch.zeros(T, dtype=torch.bool)
    runs = [(t, 1) for t in range(T)] if blocks is None else [(int(a), int(n)) for a, n in blocks.tolist()]
    for t0, n in runs:
        for t in range(t0, t0 + n):
            assert not covered[t]
            covered[t] = True
            b = t if tok_req is None else int(tok_req[t])
            assert blocks is None or int(tok_req[t0]) == b, "a run crosses two sequences"
            slots = req_to_token[int(req_pool_indices[b]), : int(positions[t]) + 1].long()
            kk, vv = k_cache[slots].float(), v_cache[slots].float()             # [n, G, d]
            for h in range(H):
                g = h // (H // G)
                s = (kk[:, g] @ q[t, h].float()) * scale * float(temp[h]) + float(bias[h])
                out[t, h] = (torch.sigmoid(s) @ vv[:, g]).to(out.dtype)
    assert bool(covered.all()), "the runs do not cover every token"
    return out


def moe_route_grouped(logits, correction, top, n_groups, keep_groups, scale):
    T, E = logits.shape
    per = E // n_groups
    s = torch.sigmoid(logits.float())
    c = s + correction.float()
    ids = torch.empty((T, top), dtype=torch.int32)
    w = torch.empty((T, top), dtype=torch.float32)
    for t in range(T):
        gs = c[t].view(n_groups, per).topk(min(2, per), dim=-1).values.sum(-1)
        kept = set(sorted(range(n_groups), key=lambda g: (-float(gs[g]), g))[:keep_groups])
        order = sorted((e for e in range(E) if e // per in kept), key=lambda e: (-float(c[t, e]), e))[:top]
        ids[t] = torch.tensor(order, dtype=torch.int32)
        sel = s[t, order]
        w[t] = sel / (sel.sum() + 1e-20) * scale
    return ids, w


def moe_router_logits(x, weight):
    return F.linear(x, weight)


def linear_tiled_supported(m, n, k, dtype, silu_mul=False):
    return False


def moe_align(expert_ids, num_experts, wide_ok=False, tiled_ok=False, block=4):
    T, top = expert_ids.shape
    flat = expert_ids.reshape(-1).tolist()
    src, tiles = [], []
    rows = torch.empty(T * top, dtype=torch.int32)
    for e in range(num_experts):
        mine = [i for i, x in enumerate(flat) if x == e]
        for n, i in enumerate(mine):
            rows[i] = len(src) + n
        pad = (-len(mine)) % block
        tiles += [e] * ((len(mine) + pad) // block)
        src += [i // top for i in mine] + [-1] * pad
    return SimpleNamespace(src_row=torch.tensor(src, dtype=torch.int32), rows=rows.view(T, top),
                           tile_expert=torch.tensor(tiles, dtype=torch.int32), n_tiles=len(tiles), block=block,
                           padded=len(src))


def moe_grouped_linear(x, w, plan, gather, gelu):
    out = torch.zeros((plan.padded, w.shape[1]), dtype=x.dtype)
    for p in range(plan.padded):
        r = int(plan.src_row[p])
        if r < 0:
            continue
        e = int(plan.tile_expert[p // plan.block])
        y = (x[r] if gather else x[p]).float() @ w[e].float().T
        if gelu:
            y = 0.5 * y * (1.0 + torch.erf(y * 0.7071067811865476))
        out[p] = y.to(x.dtype)
    return out


def gelu_tanh_mul_rows(gate, table, ids, col_off):
    z = gate.float()
    g = 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z * z * z)))
    return (g * table[ids.long(), col_off: col_off + gate.shape[1]].float()).to(gate.dtype)


# ------------------------------------------------------- pre-norm stream with parallel branches, short convolutions, delta rule,
# windowed attention with a sink.  Token-by-token restatements of what the header says of each kernel; they share nothing
# with the whole-sequence functions of oracle/gatarax_ref.py that the tests compare against.
def offset_rmsnorm(x, weight, eps, offset=1.0):
    return (x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * (offset + weight.float())).to(weight.dtype)


def branch_residual_add(x, a, wa, b=None, wb=None, s=1.0, f=None, rows=None, coef=None, eps=1e-6):
    def branch(y, w):
        y = y.float()
        return y if w is None else y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps) * w.float()
    m = branch(a, wa)
    if b is not None:
        m = m + branch(b, wb)
    m = m * s
    if f is not None:
        if rows is None:
            m = m + f.float()
        else:
            for t in range(x.shape[0]):
                for j in range(rows.shape[1]):
                    m[t] += float(coef[t, j]) * f[int(rows[t, j])].float()
    x.add_(m)
    return x


def head_rmsnorm_gate_act(o, weight, gate, eps, out_dtype, gate_act="silu"):
    T, H, dv = o.shape
    n = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps)
    if weight is not None:
        n = n * weight.float()
    g = gate.float().reshape(T, H, dv)
    return (n * (torch.sigmoid(g) if gate_act == "sigmoid" else g * torch.sigmoid(g))).reshape(T, H * dv).to(out_dtype)


def _act(z, act):
    if act == "silu":
        return z * torch.sigmoid(z)
    if act == "relu2":
        return torch.clamp(z, min=0.0) ** 2
    return z


def causal_conv(u, w1, state, req_to_state, req_pool_indices, positions, w2=None, residual=False, act="none", tok_req=None,
                seg_start=None, seg_len=None, bias=None):
    T, C = u.shape
    taps = w1.shape[1]
    outs = [torch.empty((T, C), dtype=u.dtype) for _ in range(1 if w2 is None else 2)]
    hist = None
    for t, (b, first, last) in enumerate(_segments(T, tok_req, seg_start, seg_len)):
        slot = int(req_to_state[int(req_pool_indices[b])])
        if first:
            # the inputs before this token, oldest first; nothing before position 0
            hist = [state[slot, i].clone() if int(positions[t]) - (taps - 1 - i) >= 0 else torch.zeros(C) for i in range(taps - 1)]
        hist.append(u[t].float())
        for y, w in zip(outs, (w1, w2)):
            acc = torch.zeros(C)
            for k in range(taps - 1, -1, -1):
                acc = acc + w[:, taps - 1 - k].float() * hist[len(hist) - 1 - k]
            if residual:
                acc = acc + hist[-1]
            if bias is not None and w is w1:
                acc = acc + bias.float()
            y[t] = _act(acc, act).to(u.dtype)
        hist = hist[1:]
        if last and taps > 1:
            state[slot] = torch.stack(hist)
    return outs[0] if w2 is None else tuple(outs)


def activation(x, act):
    return _act(x.float(), act).to(x.dtype).contiguous()


def gated_delta_rule(q, k, v, beta_logits, gate_logits, rate_bias, rate_log, out, state, req_to_state, req_pool_indices, positions,
                     q_scale, tok_req=None, seg_start=None, seg_len=None):
    T, G, dk = q.shape
    H = v.shape[1]
    rep = H // G
    S = None
    for t, (b, first, last) in enumerate(_segments(T, tok_req, seg_start, seg_len)):
        slot = int(req_to_state[int(req_pool_indices[b])])
        if first:
            S = torch.zeros_like(state[slot]) if int(positions[t]) == 0 else state[slot].clone()
        z = F.softplus(gate_logits[t].float() + rate_bias.float())
        z = z[:, None].expand(H, dk) if (gate_logits.shape[1] == H and rate_bias.numel() == H) else z.view(H, dk)
        a = torch.exp(-torch.exp(rate_log.float())[:, None] * z)
        beta = torch.sigmoid(beta_logits[t].float())
        kk = k[t].float().repeat_interleave(rep, 0)
        qq = q[t].float().repeat_interleave(rep, 0) * q_scale
        S = a[:, :, None] * S
        u = beta[:, None] * (v[t].float() - torch.einsum("hkv,hk->hv", S, kk))
        S = S + kk[:, :, None] * u[:, None, :]
        out[t] = torch.einsum("hkv,hk->hv", S, qq)
        if last:
            state[slot] = S
    return out


def window_attention_block_tokens(heads, kv_heads, head_dim, v_head_dim, dtype):
    return 3


def window_attention_splits(tokens, heads, kv_heads, max_len, window, dtype, pool=0):
    return 1


def pool_kv_blocks(k_cache, v_cache, pooled_k, pooled_v, req_to_token, req_pool_indices, positions, pool, pool_div=1, tok_req=None):
    for t in range(positions.numel()):
        pos = int(positions[t])
        if (pos + 1) % pool:
            continue
        b = t if tok_req is None else int(tok_req[t])
        slots = req_to_token[int(req_pool_indices[b]), pos - pool + 1: pos + 1].long()
        dst = int(slots[-1]) // pool_div
        pooled_k[dst] = (k_cache[slots].float().sum(0) / pool).to(pooled_k.dtype)
        pooled_v[dst] = (v_cache[slots].float().sum(0) / pool).to(pooled_v.dtype)


def window_attention(q, k_cache, v_cache, out, req_to_token, req_pool_indices, positions, sink, window, scale, tok_req=None,
                     blocks=None, max_run=None, num_splits=1, pool=0, pooled_k=None, pooled_v=None, pool_div=1, head_gate=None):
    T, H, d = q.shape
    G = k_cache.shape[1]
    covered = torch.zeros(T, dtype=torch.bool)
    runs = [(t, 1) for t in range(T)] if blocks is None else [(int(a), int(n)) for a, n in blocks.tolist()]
    for t0, n in runs:
        for t in range(t0, t0 + n):
            assert not covered[t]
            covered[t] = True
            b = t if tok_req is None else int(tok_req[t])
            assert blocks is None or int(tok_req[t0]) == b, "a run crosses two sequences"
            pos = int(positions[t])
            lo = max(0, pos - window + 1) if window > 0 else 0
            slots = req_to_token[int(req_pool_indices[b]), lo: pos + 1].long()
            kk, vv = k_cache[slots].float(), v_cache[slots].float()
            if pool > 0 and window > 0:
                seen = [bb for bb in range((pos + 1) // pool) if bb * pool + pool - 1 <= pos - window]
                if seen:
                    ends = req_to_token[int(req_pool_indices[b]), [bb * pool + pool - 1 for bb in seen]].long() // pool_div
                    kk, vv = torch.cat([pooled_k[ends].float(), kk]), torch.cat([pooled_v[ends].float(), vv])
            for h in range(H):
                g = h // (H // G)
                s = (kk[:, g] @ q[t, h].float()) * scale
                if sink is not None:
                    s = torch.cat([s, sink[h].float().reshape(1)])
                p = torch.softmax(s, 0)[: kk.shape[0]]
                o = p @ vv[:, g]
                if head_gate is not None:
                    o = o * torch.sigmoid(head_gate[t, h].float())
                out[t, h] = o.to(out.dtype)
    assert bool(covered.all()), "the runs do not cover every token"
    return out


def moe_route_scores(logits, correction, top, n_groups, keep_groups, scale, score_fn="sigmoid", group_best=2, renorm=True):
    T, E = logits.shape
    per = E // n_groups
    s = torch.softmax(logits.float(), -1) if score_fn == "softmax" else torch.sigmoid(logits.float())
    c = s + (correction.float() if correction is not None else 0.0)
    ids = torch.empty((T, top), dtype=torch.int32)
    w = torch.empty((T, top), dtype=torch.float32)
    for t in range(T):
        gs = c[t].view(n_groups, per).topk(min(group_best, per), dim=-1).values.sum(-1)
        kept = set(sorted(range(n_groups), key=lambda g: (-float(gs[g]), g))[:keep_groups])
        order = sorted((e for e in range(E) if e // per in kept), key=lambda e: (-float(c[t, e]), e))[:top]
        ids[t] = torch.tensor(order, dtype=torch.int32)
        sel = s[t, order]
        w[t] = (sel / (sel.sum() + 1e-20) if renorm else sel) * scale
    return ids, w
