"""Side-by-side throughput of two model designs at equal layer sizes (random weights, synthetic prompts): prefill
tokens/s of a batch of whole prompts, decode tokens/s of a static batch, and each design's hot kernels alone with the
bytes or flops their algorithm moves against the HBM3E / matrix-core peaks.  Started by `bench.py --design-compare`;
the default workload of bench.py does not pass through here.

Seturax is compared with the package's closest model, the dense DeepSeek stack (multi-head latent attention): same
width, heads, head widths, latent ranks, feed-forward width, depth and vocabulary; Seturax's window is a parameter of
the size."""
import time

import torch

HBM_PEAK = 8.0e12
MFMA_BF16_PEAK = 2.5e15

SIZES = {
    # DeepSeek-like attention geometry (16 / 32 heads of 128 + 64, latent 512, q latent 1536) on two widths
    "w2048": dict(width=2048, heads=16, nope=128, rope=64, v=128, kv_rank=512, q_rank=1536, ff=8192, layers=4, vocab=32768, window=1024),
    "w4096": dict(width=4096, heads=32, nope=128, rope=64, v=128, kv_rank=512, q_rank=1536, ff=12288, layers=4, vocab=32768, window=1024),
    "tiny": dict(width=256, heads=16, nope=128, rope=64, v=128, kv_rank=512, q_rank=192, ff=512, layers=2, vocab=2048, window=128),
}


def seturax_config(s: dict) -> dict:
    mixer = dict(heads=s["heads"], dim=s["nope"], rot_dim=s["rope"], vdim=s["v"], kv_rank=s["kv_rank"], q_rank=s["q_rank"],
                 mask=dict(size=s["window"]), rot=dict(base=10000.0, dims=s["rope"]), scale=(s["nope"] + s["rope"]) ** -0.5)
    return dict(architecture="Seturax", vocab=s["vocab"], width=s["width"], logit_scale=1.0, norm=dict(eps=1e-6),
                embedding=dict(scale=1.0, bigram=dict(buckets=65521, mul_prev=8191, mul_cur=127)),
                layers=[dict(type="latent_attention", mixer=mixer, mlp=dict(kind="dense", ff=s["ff"])) for _ in range(s["layers"])])


def deepseek_config(s: dict, dtype: str) -> dict:
    return dict(architectures=["DeepseekV3ForCausalLM"], model_type="deepseek_v3", hidden_size=s["width"],
                num_hidden_layers=s["layers"], num_attention_heads=s["heads"], q_lora_rank=s["q_rank"], kv_lora_rank=s["kv_rank"],
                qk_nope_head_dim=s["nope"], qk_rope_head_dim=s["rope"], v_head_dim=s["v"], intermediate_size=s["ff"],
                vocab_size=s["vocab"], rms_norm_eps=1e-6, rope_theta=10000.0, max_position_embeddings=16384, rope_scaling=None,
                n_routed_experts=None, first_k_dense_replace=s["layers"], tie_word_embeddings=False, torch_dtype=dtype)


def _timed(fn, reps: int, warmup: int = 2) -> float:
    """Seconds per call, device time between two events."""
    for _ in range(warmup):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / reps


def _runner(cfg: dict, dtype: str, tokens: int, reqs: int, ctx: int, graph: bool):
    from .configs.model_config import ModelConfig
    from .model_executor.model_runner import ModelRunner
    from .server_args import ServerArgs

    sa = ServerArgs(dtype=dtype, max_total_tokens=tokens, max_running_requests=reqs, context_length=ctx,
                    disable_cuda_graph=not graph, cuda_graph_bs=[reqs - 8] if graph else None, graph_capture_fallback=True)
    return ModelRunner(ModelConfig(cfg, dtype=dtype, context_length=ctx), sa)


def model_throughput(cfg: dict, dtype: str, prefill_bs: int, prefill_len: int, decode_bs: int, decode_ctx: int, steps: int,
                     graph: bool) -> dict:
    from . import bench_one_batch as bob

    ctx = max(prefill_len, decode_ctx + steps + 8) + 16
    mr = _runner(cfg, dtype, max(prefill_bs * prefill_len, decode_bs * (decode_ctx + steps + 8)) + 64, max(prefill_bs, decode_bs) + 8,
                 ctx, graph)
    vocab = mr.model_config.vocab_size

    def fresh(bs, n):
        bob.clear_pools(mr)
        return bob.prepare_synthetic_inputs_for_latency_test(bs, n, seed=0, vocab=vocab)

    times = []
    for r in range(3):
        reqs = fresh(prefill_bs, prefill_len)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        bob.extend(reqs, mr)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    prefill_s = min(times[1:])
    reqs = fresh(decode_bs, decode_ctx)
    nxt, _, batch = bob.extend(reqs, mr)
    for _ in range(4):
        nxt, _ = bob.decode(nxt, batch, mr)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        nxt, _ = bob.decode(nxt, batch, mr)
    torch.cuda.synchronize()
    decode_s = (time.perf_counter() - t0) / steps
    out = dict(prefill_tok_s=round(prefill_bs * prefill_len / prefill_s), prefill_ms=round(prefill_s * 1e3, 2),
               decode_tok_s=round(decode_bs / decode_s), decode_ms_per_step=round(decode_s * 1e3, 3),
               graph=mr.graph_runner is not None)
    del mr
    torch.cuda.empty_cache()
    return out


def attention_kernels(s: dict, bs: int, ctx: int, prefill_bs: int, prefill_len: int) -> dict:
    """The two designs' attention launches alone, bf16.  Decode: bytes = every visible cache row once per sequence.
    Prefill: flops of the form each kernel computes (absorbed: 2 (2 rank + rope) per query-key pair and head;
    expanded multi-head: 2 (nope + rope + v))."""
    from . import ops
    from .layers.rotary_embedding import rotate_half_inv_freq

    dev, dt = "cuda", torch.bfloat16
    H, rank, rope, W = s["heads"], s["kv_rank"], s["rope"], s["window"]
    R = rank + rope
    g = torch.Generator(device=dev).manual_seed(0)
    slots = bs * ctx + 8
    cache = torch.randn(slots, R, device=dev, generator=g).to(dt)
    req_to_token = (torch.arange(bs * ctx, device=dev, dtype=torch.int32) + 1).view(bs, ctx)
    rpi = torch.arange(bs, device=dev)
    qa = torch.randn(bs, H, rank, device=dev, generator=g).to(dt)
    qr = torch.randn(bs, H, rope, device=dev, generator=g).to(dt)
    out = torch.empty_like(qa)
    sink = torch.zeros(H, device=dev)
    inv_freq = rotate_half_inv_freq(10000.0, rope).to(dev)
    pos = torch.full((bs,), ctx - 1, device=dev, dtype=torch.int64)
    res = {}
    keys = min(W, ctx)
    splits = ops.latent_window_attention_splits(bs, H, rank, W, ctx - 1, dt)
    t = _timed(lambda: ops.latent_window_attention(qa, qr, cache, out, req_to_token, rpi, pos, sink, inv_freq, rope, W, 0.07,
                                                   num_splits=splits), 20)
    b = bs * keys * R * 2
    res["seturax_decode_attention"] = dict(us=round(t * 1e6, 1), keys=keys, splits=splits, gbs=round(b / t / 1e9), of_hbm_peak=round(b / t / HBM_PEAK, 3))
    # the closest model's decode attention over the same rows (no window: all ctx rows)
    q = torch.cat([qa, qr], -1).contiguous()
    o2 = torch.empty(bs, H, rank, device=dev, dtype=dt)
    seq = torch.full((bs,), keys, device=dev, dtype=torch.int64)
    nsp = max(1, min(64, (512 + bs * ((H + 15) // 16) - 1) // (bs * ((H + 15) // 16)), keys // 256))
    logits = torch.empty(bs * H * nsp * rank, device=dev, dtype=torch.float32)
    lse = torch.empty(bs * H * nsp, device=dev, dtype=torch.float32)
    tickets = torch.zeros(max(bs * H, 1024), device=dev, dtype=torch.int32)
    chunk = torch.full((1,), (keys + nsp - 1) // nsp, device=dev, dtype=torch.int32)
    t = _timed(lambda: ops.decode_attention_mla(q, cache.view(slots, 1, R), o2, req_to_token, rpi, seq, logits if nsp > 1 else None,
                                                lse if nsp > 1 else None, nsp, rank, 0.07, 0.0, tickets=tickets if nsp > 1 else None,
                                                kv_chunk_keys=chunk if nsp > 1 else None), 20)
    b = bs * keys * R * 2
    res["deepseek_decode_attention"] = dict(us=round(t * 1e6, 1), keys=keys, splits=nsp, gbs=round(b / t / 1e9), of_hbm_peak=round(b / t / HBM_PEAK, 3))
    # prefill: whole prompts, every token a query
    T = prefill_bs * prefill_len
    cache_p = torch.randn(T + 8, R, device=dev, generator=g).to(dt)
    rtt = (torch.arange(T, device=dev, dtype=torch.int32) + 1).view(prefill_bs, prefill_len)
    qa = torch.randn(T, H, rank, device=dev, generator=g).to(dt)
    qr = torch.randn(T, H, rope, device=dev, generator=g).to(dt)
    out = torch.empty_like(qa)
    posp = torch.arange(prefill_len, device=dev).repeat(prefill_bs)
    tok_req = torch.repeat_interleave(torch.arange(prefill_bs, device=dev, dtype=torch.int32), prefill_len)
    bq = ops.latent_window_attention_block_tokens(H, rank, rope, dt)
    starts = torch.arange(0, T, bq, dtype=torch.int32)
    blocks = torch.stack([starts, torch.full_like(starts, bq)], 1).to(dev)     # prefill_len is a multiple of bq here
    assert prefill_len % bq == 0
    t = _timed(lambda: ops.latent_window_attention(qa, qr, cache_p, out, rtt, torch.arange(prefill_bs, device=dev), posp, sink, inv_freq,
                                                   rope, W, 0.07, tok_req=tok_req, blocks=blocks), 5)
    pairs = prefill_bs * sum(min(p + 1, W) for p in range(prefill_len))
    fl = pairs * H * 2 * (2 * rank + rope)
    res["seturax_prefill_attention"] = dict(ms=round(t * 1e3, 3), tflops=round(fl / t / 1e12, 1), of_mfma_peak=round(fl / t / MFMA_BF16_PEAK, 3),
                                            form="absorbed, window %d" % W)
    # the closest model's prefill: expanded multi-head attention, causal, no window
    nope, vd = s["nope"], s["v"]
    qm = torch.randn(T, H, nope + rope, device=dev, generator=g).to(dt)
    km = torch.randn(T, H, nope + rope, device=dev, generator=g).to(dt)
    vm = torch.randn(T, H, vd, device=dev, generator=g).to(dt)
    om = torch.empty(T, H, vd, device=dev, dtype=dt)
    qo = torch.arange(0, T + 1, prefill_len, device=dev, dtype=torch.int32)
    kvp = torch.zeros(prefill_bs + 1, device=dev, dtype=torch.int32)
    dummy = torch.zeros(1, device=dev, dtype=torch.int32)
    t = _timed(lambda: ops.extend_attention_fwd(qm, km, vm, om, km, vm, qo, kvp, dummy, None, True, None, prefill_len, 0.07, 0.0), 5)
    pairs = prefill_bs * prefill_len * (prefill_len + 1) // 2
    fl = pairs * H * 2 * (nope + rope + vd)
    res["deepseek_prefill_attention"] = dict(ms=round(t * 1e3, 3), tflops=round(fl / t / 1e12, 1), of_mfma_peak=round(fl / t / MFMA_BF16_PEAK, 3),
                                             form="expanded multi-head, causal over %d" % prefill_len)
    return res


def stream_kernels(s: dict, tokens: int) -> dict:
    """The elementwise launches of a layer beside the closest model's like ones, by bytes moved (bf16 activations)."""
    from . import ops

    dev, dt = "cuda", torch.bfloat16
    D, ff = s["width"], s["ff"]
    g = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(tokens, D, device=dev, generator=g)
    w = torch.ones(D, device=dev, dtype=dt)
    state = torch.zeros(8, D, device=dev)
    r2s = torch.ones(tokens, device=dev, dtype=torch.int32)
    rpi = torch.arange(tokens, device=dev)
    pos = torch.arange(1, tokens + 1, device=dev)
    hl = torch.empty(tokens, D, device=dev)
    res = {}
    t = _timed(lambda: ops.layernorm_shift(x, w, 1e-6, shift=w, state=state, req_to_state=r2s, req_pool_indices=rpi, positions=pos, h_last=hl), 20)
    b = tokens * D * (4 + 4 + 2 + 2 + 4)     # x and the state row in, h and hs out, h_last out
    res["layernorm_shift"] = dict(us=round(t * 1e6, 1), gbs=round(b / t / 1e9))
    xb, rb = x.to(dt), x.to(dt)
    t = _timed(lambda: ops.fused_add_rmsnorm(xb, rb, w, 1e-6), 20)
    res["fused_add_rmsnorm (closest)"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * D * 2 * 4 / t / 1e9))
    hp = torch.randn(tokens, 2 * ff + 2 * D, device=dev, generator=g).to(dt)
    t = _timed(lambda: ops.gelu_tanh_and_mul(hp[:, :ff], hp[:, ff: 2 * ff]), 20)
    res["gelu_tanh_and_mul"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * ff * 2 * 3 / t / 1e9))
    gu = hp[:, : 2 * ff].contiguous()
    t = _timed(lambda: ops.silu_and_mul(gu), 20)
    res["silu_and_mul (closest)"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * ff * 2 * 3 / t / 1e9))
    y1, y2 = x.to(dt), x.to(dt)
    t = _timed(lambda: ops.gated_residual_add(x, hp[:, 2 * ff: 2 * ff + D], w, y1, hp[:, 2 * ff + D:], w, y2), 20)
    res["gated_residual_add"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * D * (8 + 8) / t / 1e9))
    return res


def run(size: str, dtype: str = "bfloat16", steps: int = 32, prefill_bs: int = 4, prefill_len: int = 2048, decode_bs: int = 64,
        decode_ctx: int = 1024) -> dict:
    from .model_loader.synthetic import hf_config_dict  # noqa: F401  (the package's presets stay as they are)

    s = SIZES[size]
    out = dict(size=size, shape=s, dtype=dtype, data="synthetic", workload=dict(prefill=[prefill_bs, prefill_len], decode=[decode_bs, decode_ctx], steps=steps))
    out["seturax"] = model_throughput(seturax_config(s), dtype, prefill_bs, prefill_len, decode_bs, decode_ctx, steps, graph=False)
    out["deepseek_dense"] = model_throughput(deepseek_config(s, dtype), dtype, prefill_bs, prefill_len, decode_bs, decode_ctx, steps, graph=True)
    out["deepseek_dense_eager"] = model_throughput(deepseek_config(s, dtype), dtype, prefill_bs, prefill_len, decode_bs, decode_ctx, steps, graph=False)
    out["attention"] = attention_kernels(s, decode_bs, decode_ctx, prefill_bs, prefill_len)
    out["stream_kernels_decode"] = stream_kernels(s, decode_bs)
    out["stream_kernels_prefill"] = stream_kernels(s, prefill_bs * prefill_len)
    return out


# ------------------------------------------------------------------------------------------------ Verozen beside Llama
# Verozen is compared with the package's closest model, Llama (multi-head attention with grouped key / value heads over
# per-head keys and values, RMS norms, one residual stream): same width, depth, vocabulary, attention heads and head
# width; Llama's dense feed-forward is as wide as the experts one Verozen token uses together.
VEROZEN_SIZES = {
    "vz2048": dict(width=2048, heads=16, kv_heads=4, dim=128, rec_heads=16, rec_dim=64, rec_vdim=128, experts=32, top=4, groups=4,
                   keep=2, ff=2048, layers=4, vocab=32768, side=64, norm_groups=8, gate_rank=64),
    "vz4096": dict(width=4096, heads=32, kv_heads=8, dim=128, rec_heads=32, rec_dim=64, rec_vdim=128, experts=64, top=8, groups=8,
                   keep=4, ff=1536, layers=4, vocab=32768, side=64, norm_groups=8, gate_rank=64),
    "vztiny": dict(width=320, heads=8, kv_heads=2, dim=64, rec_heads=4, rec_dim=32, rec_vdim=64, experts=12, top=2, groups=3, keep=2,
                   ff=128, layers=3, vocab=2048, side=8, norm_groups=5, gate_rank=24),
}


def verozen_config(s: dict) -> dict:
    mlp = dict(kind="moe", expert=dict(ff=s["ff"]),
               router=dict(experts=s["experts"], top=s["top"], scale=1.0, groups=dict(count=s["groups"], keep=s["keep"])))
    gla = dict(type="gla", mixer=dict(heads=s["rec_heads"], dim=s["rec_dim"], vdim=s["rec_vdim"], tau=8.0, gate_rank=s["gate_rank"]), mlp=mlp)
    att = dict(type="attention", mixer=dict(heads=s["heads"], kv_heads=s["kv_heads"], dim=s["dim"], vdim=s["dim"], scale=s["dim"] ** -0.5,
                                            rot=dict(base=10000.0, dims=s["dim"] // 2)), mlp=mlp)
    ret = dict(type="retention", mixer=dict(heads=s["rec_heads"], dim=s["rec_dim"], vdim=s["rec_vdim"],
                                            decay=[0.9 + 0.0123 * (i % 8) for i in range(s["rec_heads"])],
                                            rot=dict(base=100000.0, dims=s["rec_dim"])), mlp=mlp)
    order = [gla, att, ret, gla]
    return dict(architecture="Verozen", vocab=s["vocab"], width=s["width"], postln_alpha=2.0, norm=dict(eps=1e-6, groups=s["norm_groups"]),
                token_side=dict(dim=s["side"]), layers=[order[i % 4] for i in range(s["layers"])])


def llama_config(s: dict, dtype: str) -> dict:
    return dict(architectures=["LlamaForCausalLM"], model_type="llama", hidden_size=s["width"], num_hidden_layers=s["layers"],
                num_attention_heads=s["heads"], num_key_value_heads=s["kv_heads"], head_dim=s["dim"],
                intermediate_size=s["ff"] * s["top"], vocab_size=s["vocab"], rms_norm_eps=1e-6, rope_theta=10000.0,
                max_position_embeddings=16384, rope_scaling=None, tie_word_embeddings=False, torch_dtype=dtype, hidden_act="silu",
                attention_bias=False, mlp_bias=False)


def verozen_mixer_kernels(s: dict, bs: int, ctx: int, prefill_bs: int, prefill_len: int) -> dict:
    """The token mixers' launches alone, bf16, beside Llama's attention launches on the same heads.  Decode attention:
    bytes = every visible key and value row once per sequence.  Prefill attention: flops 2 (d + dv) per causal
    query-key pair and head.  The recurrence has no like kernel in the package: a decode step is priced by the bytes of
    the matrices it must read and write, a prefill by the fp32 vector flops it does (6 per matrix element and token)."""
    from . import ops

    dev, dt = "cuda", torch.bfloat16
    H, G, d = s["heads"], s["kv_heads"], s["dim"]
    g = torch.Generator(device=dev).manual_seed(0)
    res = {}
    # ---- decode attention
    slots = bs * ctx + 8
    kc = torch.randn(slots, G, d, device=dev, generator=g).to(dt)
    vc = torch.randn(slots, G, d, device=dev, generator=g).to(dt)
    rtt = (torch.arange(bs * ctx, device=dev, dtype=torch.int32) + 1).view(bs, ctx)
    rpi = torch.arange(bs, device=dev)
    q = torch.randn(bs, H, d, device=dev, generator=g).to(dt)
    o = torch.empty_like(q)
    temp, bias = torch.ones(H, device=dev), torch.full((H,), -4.0, device=dev)
    pos = torch.full((bs,), ctx - 1, device=dev, dtype=torch.int64)
    splits = ops.sigmoid_attention_splits(bs, H, G, ctx, dt)
    t = _timed(lambda: ops.sigmoid_attention(q, kc, vc, o, rtt, rpi, pos, temp, bias, d ** -0.5, num_splits=splits), 20)
    b = bs * ctx * G * d * 2 * 2
    res["verozen_decode_attention"] = dict(us=round(t * 1e6, 1), splits=splits, gbs=round(b / t / 1e9), of_hbm_peak=round(b / t / HBM_PEAK, 3))
    seq = torch.full((bs,), ctx, device=dev, dtype=torch.int64)
    nsp = int(ops.decode_num_splits(bs, G, ctx, 64))
    logits = torch.empty(bs * H * nsp * d, device=dev, dtype=torch.float32)
    lse = torch.empty(bs * H * nsp, device=dev, dtype=torch.float32)
    o2 = torch.empty(bs, H, d, device=dev, dtype=dt)
    t = _timed(lambda: ops.decode_attention_paged(q, kc, vc, o2, rtt, rpi, seq, logits if nsp > 1 else None, lse if nsp > 1 else None,
                                                  nsp, d ** -0.5), 20)
    res["llama_decode_attention"] = dict(us=round(t * 1e6, 1), splits=nsp, gbs=round(b / t / 1e9), of_hbm_peak=round(b / t / HBM_PEAK, 3))
    # ---- prefill attention
    T = prefill_bs * prefill_len
    kp = torch.randn(T + 8, G, d, device=dev, generator=g).to(dt)
    vp = torch.randn(T + 8, G, d, device=dev, generator=g).to(dt)
    rtp = (torch.arange(T, device=dev, dtype=torch.int32) + 1).view(prefill_bs, prefill_len)
    qp = torch.randn(T, H, d, device=dev, generator=g).to(dt)
    op = torch.empty_like(qp)
    posp = torch.arange(prefill_len, device=dev).repeat(prefill_bs)
    tok_req = torch.repeat_interleave(torch.arange(prefill_bs, device=dev, dtype=torch.int32), prefill_len)
    bq = ops.sigmoid_attention_block_tokens(H, G, d, d, dt)
    assert prefill_len % bq == 0
    starts = torch.arange(0, T, bq, dtype=torch.int32)
    blocks = torch.stack([starts, torch.full_like(starts, bq)], 1).to(dev)
    t = _timed(lambda: ops.sigmoid_attention(qp, kp, vp, op, rtp, torch.arange(prefill_bs, device=dev), posp, temp, bias, d ** -0.5,
                                             tok_req=tok_req, blocks=blocks, max_run=bq), 3)
    pairs = prefill_bs * prefill_len * (prefill_len + 1) // 2
    fl = pairs * H * 2 * 2 * d
    res["verozen_prefill_attention"] = dict(ms=round(t * 1e3, 3), tflops=round(fl / t / 1e12, 1), of_mfma_peak=round(fl / t / MFMA_BF16_PEAK, 3))
    km = torch.randn(T, G, d, device=dev, generator=g).to(dt)
    vm = torch.randn(T, G, d, device=dev, generator=g).to(dt)
    qo = torch.arange(0, T + 1, prefill_len, device=dev, dtype=torch.int32)
    kvp = torch.zeros(prefill_bs + 1, device=dev, dtype=torch.int32)
    dummy = torch.zeros(1, device=dev, dtype=torch.int32)
    t = _timed(lambda: ops.extend_attention_fwd(qp, km, vm, op, km, vm, qo, kvp, dummy, None, True, None, prefill_len, d ** -0.5, 0.0), 5)
    res["llama_prefill_attention"] = dict(ms=round(t * 1e3, 3), tflops=round(fl / t / 1e12, 1), of_mfma_peak=round(fl / t / MFMA_BF16_PEAK, 3))
    # ---- the recurrence
    RH, dk, dv = s["rec_heads"], s["rec_dim"], s["rec_vdim"]
    state = torch.zeros(bs + 1, RH, dk, dv, device=dev)
    r2s = torch.arange(1, bs + 1, device=dev, dtype=torch.int32)
    for name, gated in (("gla", True), ("retention", False)):
        qk_dt = dt if gated else torch.float32
        qd = torch.randn(bs, RH, dk, device=dev, generator=g).to(qk_dt)
        kd = torch.randn(bs, RH, dk, device=dev, generator=g).to(qk_dt)
        vd = torch.randn(bs, RH, dv, device=dev, generator=g).to(dt)
        od = torch.empty(bs, RH, dv, device=dev)
        z = torch.randn(bs, RH * dk, device=dev, generator=g) if gated else None
        hd = None if gated else torch.full((RH,), 0.99, device=dev)
        posd = torch.full((bs,), ctx, device=dev, dtype=torch.int64)
        t = _timed(lambda: ops.linear_recurrence(qd, kd, vd, od, state, r2s, rpi, posd, 1.0, gate_logits=z, tau=8.0, head_decay=hd), 20)
        b = bs * RH * dk * dv * 4 * 2
        res[f"verozen_{name}_decode_recurrence"] = dict(us=round(t * 1e6, 1), gbs=round(b / t / 1e9), of_hbm_peak=round(b / t / HBM_PEAK, 3))
        qd = torch.randn(T, RH, dk, device=dev, generator=g).to(qk_dt)
        kd = torch.randn(T, RH, dk, device=dev, generator=g).to(qk_dt)
        vd = torch.randn(T, RH, dv, device=dev, generator=g).to(dt)
        od = torch.empty(T, RH, dv, device=dev)
        z = torch.randn(T, RH * dk, device=dev, generator=g) if gated else None
        ss = torch.arange(0, T, prefill_len, device=dev, dtype=torch.int32)
        sl = torch.full((prefill_bs,), prefill_len, device=dev, dtype=torch.int32)
        t = _timed(lambda: ops.linear_recurrence(qd, kd, vd, od, state, r2s, torch.arange(prefill_bs, device=dev), posp, 1.0,
                                                 gate_logits=z, tau=8.0, head_decay=hd, tok_req=tok_req, seg_start=ss, seg_len=sl), 3)
        fl = T * RH * dk * dv * 6
        res[f"verozen_{name}_prefill_recurrence"] = dict(ms=round(t * 1e3, 3), vector_tflops=round(fl / t / 1e12, 2),
                                                          tokens_per_s_per_sequence=round(prefill_len / t))
    return res


def verozen_ff_and_stream_kernels(s: dict, tokens: int) -> dict:
    """The mixture's launches beside Llama's dense feed-forward GEMMs at equal flops per token, and the post-norm
    launches beside fused_add_rmsnorm by bytes moved (bf16 activations)."""
    import torch.nn.functional as F

    from . import ops

    dev, dt = "cuda", torch.bfloat16
    D, ff, E, top = s["width"], s["ff"], s["experts"], s["top"]
    g = torch.Generator(device=dev).manual_seed(0)
    res = {}
    x = torch.randn(tokens, D, device=dev, generator=g)
    h = x.to(dt)
    wr = torch.randn(E, D, device=dev, generator=g) * D ** -0.5
    corr = torch.zeros(E, device=dev)
    up = (torch.randn(E, ff, D, device=dev, generator=g) * D ** -0.5).to(dt)
    down = (torch.randn(E, D, ff, device=dev, generator=g) * ff ** -0.5).to(dt)
    logits = ops.moe_router_logits(x, wr)
    t = _timed(lambda: ops.moe_router_logits(x, wr), 10)
    res["router_logits_fp32"] = dict(us=round(t * 1e6, 1))
    ids, wts = ops.moe_route_grouped(logits, corr, top, s["groups"], s["keep"], 1.0)
    t = _timed(lambda: ops.moe_route_grouped(logits, corr, top, s["groups"], s["keep"], 1.0), 10)
    res["moe_route_grouped"] = dict(us=round(t * 1e6, 1))
    plan = ops.moe_align(ids, E, wide_ok=True, tiled_ok=tokens > 64)
    t = _timed(lambda: ops.moe_align(ids, E, wide_ok=True, tiled_ok=tokens > 64), 10)
    res["moe_align"] = dict(us=round(t * 1e6, 1))
    a = ops.moe_grouped_linear(h, up, plan, gather=True, gelu=True)
    t1 = _timed(lambda: ops.moe_grouped_linear(h, up, plan, gather=True, gelu=True), 5)
    t2 = _timed(lambda: ops.moe_grouped_linear(a, down, plan, gather=False, gelu=False), 5)
    fl = tokens * top * 2 * ff * D
    wbytes = E * ff * D * 2
    res["moe_block_rows"] = plan.block
    res["moe_up_gelu"] = dict(us=round(t1 * 1e6, 1), tflops=round(fl / t1 / 1e12, 1), of_mfma_peak=round(fl / t1 / MFMA_BF16_PEAK, 3),
                              weight_gbs=round(wbytes / t1 / 1e9))
    res["moe_down"] = dict(us=round(t2 * 1e6, 1), tflops=round(fl / t2 / 1e12, 1), of_mfma_peak=round(fl / t2 / MFMA_BF16_PEAK, 3),
                           weight_gbs=round(wbytes / t2 / 1e9))
    # the closest model's feed-forward: one [ff * top, D] up projection (half of gate_up) and the down projection
    wu = (torch.randn(ff * top, D, device=dev, generator=g) * D ** -0.5).to(dt)
    wd = (torch.randn(D, ff * top, device=dev, generator=g) * (ff * top) ** -0.5).to(dt)
    mid = torch.randn(tokens, ff * top, device=dev, generator=g).to(dt)
    t1 = _timed(lambda: F.linear(h, wu), 5)
    t2 = _timed(lambda: F.linear(mid, wd), 5)
    res["dense_up (closest, library GEMM)"] = dict(us=round(t1 * 1e6, 1), tflops=round(fl / t1 / 1e12, 1), of_mfma_peak=round(fl / t1 / MFMA_BF16_PEAK, 3),
                                                    weight_gbs=round(ff * top * D * 2 / t1 / 1e9))
    res["dense_down (closest, library GEMM)"] = dict(us=round(t2 * 1e6, 1), tflops=round(fl / t2 / 1e12, 1), of_mfma_peak=round(fl / t2 / MFMA_BF16_PEAK, 3),
                                                      weight_gbs=round(ff * top * D * 2 / t2 / 1e9))
    # norms
    w = torch.ones(D, device=dev, dtype=dt)
    y = torch.randn(tokens, D, device=dev, generator=g).to(dt)
    t = _timed(lambda: ops.scaled_add_group_rmsnorm(x, y, 3.0, w, s["norm_groups"], 1e-5), 20)
    res["scaled_add_group_rmsnorm"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * D * (4 + 2 + 4 + 2) / t / 1e9))
    yy = ops.moe_grouped_linear(a, down, plan, gather=False, gelu=False)
    t = _timed(lambda: ops.scaled_add_group_rmsnorm(x, yy, 3.0, w, s["norm_groups"], 1e-5, rows=plan.rows, coef=wts), 20)
    res["scaled_add_group_rmsnorm (sum of experts)"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * D * (4 + 2 * top + 4 + 2) / t / 1e9))
    t = _timed(lambda: ops.rmsnorm_residual_add(x, y, w, 1e-5), 20)
    res["rmsnorm_residual_add"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * D * (4 + 2 + 4 + 2) / t / 1e9))
    xb, rb = x.to(dt), x.to(dt)
    t = _timed(lambda: ops.fused_add_rmsnorm(xb, rb, w, 1e-5), 20)
    res["fused_add_rmsnorm (closest)"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * D * 2 * 4 / t / 1e9))
    return res


def run_verozen(size: str, dtype: str = "bfloat16", steps: int = 32, prefill_bs: int = 4, prefill_len: int = 2048, decode_bs: int = 64,
                decode_ctx: int = 1024) -> dict:
    s = VEROZEN_SIZES[size]
    if size == "vztiny":
        prefill_bs, prefill_len, decode_bs, decode_ctx = 2, 256, 8, 128
    out = dict(size=size, shape=s, dtype=dtype, data="synthetic", workload=dict(prefill=[prefill_bs, prefill_len], decode=[decode_bs, decode_ctx], steps=steps))
    out["verozen"] = model_throughput(verozen_config(s), dtype, prefill_bs, prefill_len, decode_bs, decode_ctx, steps, graph=False)
    out["llama"] = model_throughput(llama_config(s, dtype), dtype, prefill_bs, prefill_len, decode_bs, decode_ctx, steps, graph=True)
    out["llama_eager"] = model_throughput(llama_config(s, dtype), dtype, prefill_bs, prefill_len, decode_bs, decode_ctx, steps, graph=False)
    out["mixers"] = verozen_mixer_kernels(s, decode_bs, decode_ctx, prefill_bs, prefill_len)
    out["ff_and_stream_decode"] = verozen_ff_and_stream_kernels(s, decode_bs)
    out["ff_and_stream_prefill"] = verozen_ff_and_stream_kernels(s, prefill_bs * prefill_len)
    return out


# ------------------------------------------------------------------------------------------------ Gatarax beside Verozen
# Gatarax is compared with the package's closest model, Verozen (an fp32 residual stream, attention with grouped key heads
# over per-layer caches beside recurrent mixers with a matrix per head and sequence, a grouped mixture of experts): same
# width, depth, vocabulary, attention heads and head widths, recurrent heads, experts and expert width.
GATARAX_SIZES = {
    "gx2048": dict(VEROZEN_SIZES["vz2048"], window=1024, taps=4, conv=4, rec_kv_heads=16, low_rank=64),
    "gx4096": dict(VEROZEN_SIZES["vz4096"], window=1024, taps=4, conv=4, rec_kv_heads=32, low_rank=64),
    "gxtiny": dict(VEROZEN_SIZES["vztiny"], window=96, taps=4, conv=3, rec_kv_heads=2, low_rank=24),
}


def gatarax_config(s: dict) -> dict:
    mlp = dict(kind="moe", expert=dict(ff=s["ff"]), router=dict(experts=s["experts"], top=s["top"], groups=dict(count=s["groups"], keep=s["keep"])))
    par = dict(type="parallel", mlp=mlp,
               mixer=dict(left=dict(heads=s["heads"], kv_heads=s["kv_heads"], dim=s["dim"], vdim=s["dim"], conv=s["conv"], scale=s["dim"] ** -0.5,
                                    mask=dict(size=s["window"])),
                          right=dict(heads=s["rec_heads"], kv_heads=s["rec_kv_heads"], dim=s["rec_dim"], vdim=s["rec_vdim"], conv=s["conv"],
                                     decay_rank=s["low_rank"], gate_rank=s["low_rank"])))
    lit = dict(type="lightning", mlp=mlp, mixer=dict(heads=s["rec_heads"], dim=s["rec_dim"], vdim=s["rec_vdim"],
                                                     decay=[0.9 + 0.0123 * (i % 8) for i in range(s["rec_heads"])]))
    order = [par, lit, par, lit]
    return dict(architecture="Gatarax", vocab=s["vocab"], width=s["width"], logit_scale=1.0, norm=dict(eps=1e-6), embedding=dict(scale=1.0),
                canon=dict(taps=s["taps"]), layers=[order[i % 4] for i in range(s["layers"])])


def gatarax_mixer_kernels(s: dict, bs: int, ctx: int, prefill_bs: int, prefill_len: int) -> dict:
    """The token mixers' launches alone, bf16, each beside the closest model's like launch on the same shapes: windowed
    softmax attention beside sigmoid attention (decode: bytes = every visible key and value row once per sequence; prefill:
    flops 2 (d + dv) per visible query-key pair and head), the gated delta rule beside the gated linear recurrence (decode:
    the matrices' bytes, read and written; prefill: fp32 vector flops, 6 per matrix element and token for the plain
    recurrence, 10 for the delta rule)."""
    from . import ops

    dev, dt = "cuda", torch.bfloat16
    H, G, d, W = s["heads"], s["kv_heads"], s["dim"], s["window"]
    g = torch.Generator(device=dev).manual_seed(0)
    res = {}
    slots = bs * ctx + 8
    kc = torch.randn(slots, G, d, device=dev, generator=g).to(dt)
    vc = torch.randn(slots, G, d, device=dev, generator=g).to(dt)
    rtt = (torch.arange(bs * ctx, device=dev, dtype=torch.int32) + 1).view(bs, ctx)
    rpi = torch.arange(bs, device=dev)
    q = torch.randn(bs, H, d, device=dev, generator=g).to(dt)
    o = torch.empty_like(q)
    sink = torch.zeros(H, device=dev)
    pos = torch.full((bs,), ctx - 1, device=dev, dtype=torch.int64)
    wsplits = ops.window_attention_splits(bs, H, G, ctx, W, dt)
    t = _timed(lambda: ops.window_attention(q, kc, vc, o, rtt, rpi, pos, sink, W, d ** -0.5, num_splits=wsplits), 20)
    b = bs * min(ctx, W) * G * d * 2 * 2
    res["gatarax_decode_attention"] = dict(us=round(t * 1e6, 1), splits=wsplits, gbs=round(b / t / 1e9), of_hbm_peak=round(b / t / HBM_PEAK, 3))
    temp, bias = torch.ones(H, device=dev), torch.full((H,), -4.0, device=dev)
    splits = ops.sigmoid_attention_splits(bs, H, G, ctx, dt)
    t = _timed(lambda: ops.sigmoid_attention(q, kc, vc, o, rtt, rpi, pos, temp, bias, d ** -0.5, num_splits=splits), 20)
    b = bs * ctx * G * d * 2 * 2
    res["verozen_decode_attention"] = dict(us=round(t * 1e6, 1), splits=splits, gbs=round(b / t / 1e9), of_hbm_peak=round(b / t / HBM_PEAK, 3))
    # ---- prefill attention
    T = prefill_bs * prefill_len
    kp = torch.randn(T + 8, G, d, device=dev, generator=g).to(dt)
    vp = torch.randn(T + 8, G, d, device=dev, generator=g).to(dt)
    rtp = (torch.arange(T, device=dev, dtype=torch.int32) + 1).view(prefill_bs, prefill_len)
    qp = torch.randn(T, H, d, device=dev, generator=g).to(dt)
    op = torch.empty_like(qp)
    posp = torch.arange(prefill_len, device=dev).repeat(prefill_bs)
    tok_req = torch.repeat_interleave(torch.arange(prefill_bs, device=dev, dtype=torch.int32), prefill_len)
    rpp = torch.arange(prefill_bs, device=dev)
    bq = ops.window_attention_block_tokens(H, G, d, d, dt)
    assert prefill_len % bq == 0
    starts = torch.arange(0, T, bq, dtype=torch.int32)
    blocks = torch.stack([starts, torch.full_like(starts, bq)], 1).to(dev)
    t = _timed(lambda: ops.window_attention(qp, kp, vp, op, rtp, rpp, posp, sink, W, d ** -0.5, tok_req=tok_req, blocks=blocks, max_run=bq), 3)
    pairs = prefill_bs * sum(min(i + 1, W) for i in range(prefill_len))
    fl = pairs * H * 2 * 2 * d
    res["gatarax_prefill_attention"] = dict(ms=round(t * 1e3, 3), tflops=round(fl / t / 1e12, 1), of_mfma_peak=round(fl / t / MFMA_BF16_PEAK, 3))
    bq2 = ops.sigmoid_attention_block_tokens(H, G, d, d, dt)
    starts = torch.arange(0, T, bq2, dtype=torch.int32)
    blocks2 = torch.stack([starts, torch.full_like(starts, bq2)], 1).to(dev)
    t = _timed(lambda: ops.sigmoid_attention(qp, kp, vp, op, rtp, rpp, posp, temp, bias, d ** -0.5, tok_req=tok_req, blocks=blocks2, max_run=bq2), 3)
    fl = prefill_bs * prefill_len * (prefill_len + 1) // 2 * H * 2 * 2 * d
    res["verozen_prefill_attention"] = dict(ms=round(t * 1e3, 3), tflops=round(fl / t / 1e12, 1), of_mfma_peak=round(fl / t / MFMA_BF16_PEAK, 3))
    # ---- the recurrences
    RH, RG, dk, dv = s["rec_heads"], s["rec_kv_heads"], s["rec_dim"], s["rec_vdim"]
    state = torch.zeros(bs + 1, RH, dk, dv, device=dev)
    r2s = torch.arange(1, bs + 1, device=dev, dtype=torch.int32)
    rb, rl = torch.zeros(RH * dk, device=dev), torch.zeros(RH, device=dev)
    ss = torch.arange(0, T, prefill_len, device=dev, dtype=torch.int32)
    sl = torch.full((prefill_bs,), prefill_len, device=dev, dtype=torch.int32)
    for n, seg, reps in ((bs, {}, 20), (T, dict(tok_req=tok_req, seg_start=ss, seg_len=sl), 3)):
        qd = torch.nn.functional.normalize(torch.randn(n, RG, dk, device=dev, generator=g), dim=-1)
        kd = torch.nn.functional.normalize(torch.randn(n, RG, dk, device=dev, generator=g), dim=-1)
        vd = torch.randn(n, RH, dv, device=dev, generator=g).to(dt)
        be = torch.randn(n, RH, device=dev, generator=g).to(dt)
        z = torch.randn(n, RH * dk, device=dev, generator=g)
        od = torch.empty(n, RH, dv, device=dev)
        rp_, ps_ = (rpi, torch.full((bs,), ctx, device=dev, dtype=torch.int64)) if not seg else (rpp, posp)
        t = _timed(lambda: ops.gated_delta_rule(qd, kd, vd, be, z, rb, rl, od, state, r2s, rp_, ps_, dk ** -0.5, **seg), reps)
        qg, kg = (torch.randn(n, RH, dk, device=dev, generator=g).to(dt) for _ in range(2))
        t2 = _timed(lambda: ops.linear_recurrence(qg, kg, vd, od, state, r2s, rp_, ps_, 1.0, gate_logits=z, tau=8.0, **seg), reps)
        if not seg:
            b = bs * RH * dk * dv * 4 * 2
            res["gatarax_delta_rule_decode"] = dict(us=round(t * 1e6, 1), gbs=round(b / t / 1e9), of_hbm_peak=round(b / t / HBM_PEAK, 3))
            res["verozen_gla_decode_recurrence"] = dict(us=round(t2 * 1e6, 1), gbs=round(b / t2 / 1e9), of_hbm_peak=round(b / t2 / HBM_PEAK, 3))
        else:
            res["gatarax_delta_rule_prefill"] = dict(ms=round(t * 1e3, 3), vector_tflops=round(T * RH * dk * dv * 10 / t / 1e12, 2),
                                                     tokens_per_s_per_sequence=round(prefill_len / t))
            res["verozen_gla_prefill_recurrence"] = dict(ms=round(t2 * 1e3, 3), vector_tflops=round(T * RH * dk * dv * 6 / t2 / 1e12, 2),
                                                         tokens_per_s_per_sequence=round(prefill_len / t2))
    return res


def gatarax_stream_kernels(s: dict, tokens: int, segments: int) -> dict:
    """The elementwise launches by bytes moved (bf16 activations, fp32 stream) beside the closest model's norm launch, and
    the experts' first GEMM with its activation (one launch with erf-GELU there, a GEMM twice as wide plus silu-and-mul here)."""
    from . import ops

    dev, dt = "cuda", torch.bfloat16
    D, ff, E, top = s["width"], s["ff"], s["experts"], s["top"]
    g = torch.Generator(device=dev).manual_seed(0)
    res = {}
    x = torch.randn(tokens, D, device=dev, generator=g)
    w = torch.ones(D, device=dev, dtype=dt)
    t = _timed(lambda: ops.offset_rmsnorm(x, w, 1e-6, 1.0), 20)
    res["offset_rmsnorm"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * D * (4 + 2) / t / 1e9))
    h = x.to(dt)
    taps = s["taps"]
    w1, w2 = (torch.randn(D, taps, device=dev, generator=g).to(dt) for _ in range(2))
    state = torch.zeros(segments + 1, taps - 1, D, device=dev)
    r2s = torch.arange(1, segments + 1, device=dev, dtype=torch.int32)
    rpi = torch.arange(segments, device=dev)
    per = tokens // segments
    if per == 1:
        seg, pos = {}, torch.full((tokens,), 100, device=dev, dtype=torch.int64)
    else:
        seg = dict(tok_req=torch.repeat_interleave(torch.arange(segments, device=dev, dtype=torch.int32), per),
                   seg_start=torch.arange(0, tokens, per, device=dev, dtype=torch.int32),
                   seg_len=torch.full((segments,), per, device=dev, dtype=torch.int32))
        pos = torch.arange(per, device=dev).repeat(segments)
    t = _timed(lambda: ops.causal_conv(h, w1, state, r2s, rpi, pos, w2=w2, residual=True, **seg), 20)
    res["causal_conv (two filters, with the state's update)"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * D * 2 * 3 / t / 1e9))
    a, b, f = (torch.randn(tokens, D, device=dev, generator=g).to(dt) for _ in range(3))
    t = _timed(lambda: ops.branch_residual_add(x, a, w, b, w, 0.5, f=f), 20)
    res["branch_residual_add (two normed branches, dense ff)"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * D * (4 + 4 + 3 * 2) / t / 1e9))
    big = torch.randn(tokens * top, D, device=dev, generator=g).to(dt)
    rows = torch.randperm(tokens * top, device=dev, generator=g).to(torch.int32).view(tokens, top)
    coef = torch.rand(tokens, top, device=dev, generator=g)
    t = _timed(lambda: ops.branch_residual_add(x, a, w, b, w, 0.5, f=big, rows=rows, coef=coef), 20)
    res["branch_residual_add (two normed branches, sum of experts)"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * D * (4 + 4 + (2 + top) * 2) / t / 1e9))
    t = _timed(lambda: ops.scaled_add_group_rmsnorm(x, f, 3.0, w, s["norm_groups"], 1e-5), 20)
    res["scaled_add_group_rmsnorm (closest)"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * D * (4 + 2 + 4 + 2) / t / 1e9))
    # experts: first GEMM + activation
    ids, _ = ops.moe_route_scores(torch.randn(tokens, E, device=dev, generator=g), None, top, s["groups"], s["keep"], 1.0, score_fn="softmax",
                                  group_best=1, renorm=False)
    t = _timed(lambda: ops.moe_route_scores(torch.zeros(tokens, E, device=dev), None, top, s["groups"], s["keep"], 1.0, score_fn="softmax",
                                            group_best=1, renorm=False), 10)
    res["moe_route_scores (softmax; with the fill of its input)"] = dict(us=round(t * 1e6, 1))
    plan = ops.moe_align(ids, E, wide_ok=True, tiled_ok=tokens > 64)
    gu_w = (torch.randn(E, 2 * ff, D, device=dev, generator=g) * D ** -0.5).to(dt)
    up = gu_w[:, :ff].contiguous()
    t1 = _timed(lambda: ops.silu_and_mul(ops.moe_grouped_linear(h, gu_w, plan, gather=True, gelu=False)), 5)
    t2 = _timed(lambda: ops.moe_grouped_linear(h, up, plan, gather=True, gelu=True), 5)
    fl = tokens * top * 2 * ff * D
    res["moe_block_rows"] = plan.block
    res["moe_gate_up_silu_mul"] = dict(us=round(t1 * 1e6, 1), tflops=round(2 * fl / t1 / 1e12, 1), of_mfma_peak=round(2 * fl / t1 / MFMA_BF16_PEAK, 3),
                                       weight_gbs=round(2 * E * ff * D * 2 / t1 / 1e9))
    res["moe_up_gelu (closest)"] = dict(us=round(t2 * 1e6, 1), tflops=round(fl / t2 / 1e12, 1), of_mfma_peak=round(fl / t2 / MFMA_BF16_PEAK, 3),
                                        weight_gbs=round(E * ff * D * 2 / t2 / 1e9))
    return res


def run_gatarax(size: str, dtype: str = "bfloat16", steps: int = 32, prefill_bs: int = 4, prefill_len: int = 2048, decode_bs: int = 64,
                decode_ctx: int = 1024) -> dict:
    s = GATARAX_SIZES[size]
    if size == "gxtiny":
        prefill_bs, prefill_len, decode_bs, decode_ctx = 2, 256, 8, 128
    out = dict(size=size, shape=s, dtype=dtype, data="synthetic", workload=dict(prefill=[prefill_bs, prefill_len], decode=[decode_bs, decode_ctx], steps=steps))
    out["gatarax"] = model_throughput(gatarax_config(s), dtype, prefill_bs, prefill_len, decode_bs, decode_ctx, steps, graph=False)
    out["verozen"] = model_throughput(verozen_config(s), dtype, prefill_bs, prefill_len, decode_bs, decode_ctx, steps, graph=False)
    out["mixers"] = gatarax_mixer_kernels(s, decode_bs, decode_ctx, prefill_bs, prefill_len)
    out["stream_decode"] = gatarax_stream_kernels(s, decode_bs, decode_bs)
    out["stream_prefill"] = gatarax_stream_kernels(s, prefill_bs * prefill_len, prefill_bs)
    return out


# ------------------------------------------------------------------------------------------------ Fudonex beside Gatarax
# Fudonex is compared with the package's closest model, Gatarax (an fp32 residual stream, windowed softmax attention with a
# sink over per-layer caches, a gated delta rule and a linear recurrence with a matrix per head and sequence, short causal
# convolutions with state): same width, depth, vocabulary, attention heads and head widths, window, recurrent heads and
# widths.  Both run dense feed-forwards here, of equal weight count (gated: three matrices of ff; ungated: two of 1.5 ff).
FUDONEX_SIZES = {
    "fx2048": dict(width=2048, heads=16, kv_heads=4, dim=128, rec_heads=16, rec_kv_heads=16, rec_dim=64, rec_vdim=128, groups=4, norm_groups=4,
                   ff=5632, layers=4, vocab=32768, window=512, pool=64, conv=4, rot=64),
    "fx4096": dict(width=4096, heads=32, kv_heads=8, dim=128, rec_heads=32, rec_kv_heads=32, rec_dim=64, rec_vdim=128, groups=8, norm_groups=8,
                   ff=11264, layers=4, vocab=32768, window=512, pool=64, conv=4, rot=64),
    "fxtiny": dict(width=320, heads=8, kv_heads=2, dim=64, rec_heads=4, rec_kv_heads=2, rec_dim=32, rec_vdim=64, groups=2, norm_groups=2,
                   ff=512, layers=4, vocab=2048, window=64, pool=16, conv=3, rot=32),
}


def fudonex_config(s: dict) -> dict:
    mlp = dict(kind="dense", ff=s["ff"])
    att = dict(heads=s["heads"], kv_heads=s["kv_heads"], dim=s["dim"], vdim=s["dim"], scale=s["dim"] ** -0.5,
               mask=dict(size=s["window"], pool=s["pool"]),
               rot=dict(base=10000.0, dims=s["rot"], scaling=dict(factor=4.0, original=2048, fast=16.0, slow=2.0)))
    order = [dict(type="attention", mixer=att, mlp=mlp),
             dict(type="mamba2", mlp=mlp, mixer=dict(heads=s["rec_heads"], vdim=s["rec_vdim"], state=s["rec_dim"], groups=s["groups"],
                                                     norm_groups=s["norm_groups"], conv=s["conv"])),
             dict(type="delta", mlp=mlp, mixer=dict(heads=s["rec_heads"], kv_heads=s["rec_kv_heads"], dim=s["rec_dim"], vdim=s["rec_vdim"],
                                                    conv=s["conv"])),
             dict(type="attention", mixer=dict(att, kv_from=0), mlp=mlp)]
    return dict(architecture="Fudonex", vocab=s["vocab"], width=s["width"], norm=dict(eps=1e-6), embedding=dict(scale=1.0), residual_mult=0.5,
                logit_softcap=30.0, layers=[order[i % 4] for i in range(s["layers"])])


def gatarax_dense_config(s: dict) -> dict:
    mlp = dict(kind="dense", ff=s["ff"] * 3 // 2)
    par = dict(type="parallel", mlp=mlp,
               mixer=dict(left=dict(heads=s["heads"], kv_heads=s["kv_heads"], dim=s["dim"], vdim=s["dim"], conv=s["conv"], scale=s["dim"] ** -0.5,
                                    mask=dict(size=s["window"])),
                          right=dict(heads=s["rec_heads"], kv_heads=s["rec_kv_heads"], dim=s["rec_dim"], vdim=s["rec_vdim"], conv=s["conv"],
                                     decay_rank=64, gate_rank=64)))
    lit = dict(type="lightning", mlp=mlp, mixer=dict(heads=s["rec_heads"], dim=s["rec_dim"], vdim=s["rec_vdim"],
                                                     decay=[0.9 + 0.0123 * (i % 8) for i in range(s["rec_heads"])]))
    order = [par, lit, par, lit]
    return dict(architecture="Gatarax", vocab=s["vocab"], width=s["width"], logit_scale=1.0, norm=dict(eps=1e-6), embedding=dict(scale=1.0),
                canon=dict(taps=s["conv"]), layers=[order[i % 4] for i in range(s["layers"])])


def fudonex_mixer_kernels(s: dict, bs: int, ctx: int, prefill_bs: int, prefill_len: int) -> dict:
    """The token mixers' launches alone, bf16, each beside the closest model's like launch on the same shapes.  Attention:
    the same kernel with and without averaged blocks and the head gate (decode: bytes = every visible key and value row
    once per sequence, the window's and the blocks'; prefill: flops 2 (d + dv) per visible query-key or query-block pair and
    head), and the launch that writes the averages.  Recurrences: the state-space form beside the recurrence with a fixed
    decay per head, the delta rule with a decay per head beside the one with a decay per key channel (decode: the matrices'
    bytes, read and written; prefill: fp32 vector flops, 6 / 10 per matrix element and token)."""
    from . import ops

    dev, dt = "cuda", torch.bfloat16
    H, G, d, W, P = s["heads"], s["kv_heads"], s["dim"], s["window"], s["pool"]
    g = torch.Generator(device=dev).manual_seed(0)
    res = {}
    slots = bs * ctx + 8
    kc = torch.randn(slots, G, d, device=dev, generator=g).to(dt)
    vc = torch.randn(slots, G, d, device=dev, generator=g).to(dt)
    pk, pv = torch.randn_like(kc), torch.randn_like(vc)
    rtt = (torch.arange(bs * ctx, device=dev, dtype=torch.int32) + 1).view(bs, ctx)
    rpi = torch.arange(bs, device=dev)
    q = torch.randn(bs, H, d, device=dev, generator=g).to(dt)
    gate = torch.randn(bs, H, device=dev, generator=g).to(dt)
    o = torch.empty_like(q)
    sink = torch.zeros(H, device=dev)
    pos = torch.full((bs,), ctx - 1, device=dev, dtype=torch.int64)
    nblk = max(0, (ctx - 1 - W + 1) // P)
    sp = ops.window_attention_splits(bs, H, G, ctx, W, dt, pool=P)
    t = _timed(lambda: ops.window_attention(q, kc, vc, o, rtt, rpi, pos, sink, W, d ** -0.5, num_splits=sp, pool=P, pooled_k=pk, pooled_v=pv,
                                            head_gate=gate), 20)
    b = bs * (min(ctx, W) + nblk) * G * d * 2 * 2
    res["fudonex_decode_attention"] = dict(us=round(t * 1e6, 1), splits=sp, keys=min(ctx, W) + nblk, gbs=round(b / t / 1e9),
                                           of_hbm_peak=round(b / t / HBM_PEAK, 3))
    sp2 = ops.window_attention_splits(bs, H, G, ctx, W, dt)
    t = _timed(lambda: ops.window_attention(q, kc, vc, o, rtt, rpi, pos, sink, W, d ** -0.5, num_splits=sp2), 20)
    b = bs * min(ctx, W) * G * d * 2 * 2
    res["gatarax_decode_attention"] = dict(us=round(t * 1e6, 1), splits=sp2, keys=min(ctx, W), gbs=round(b / t / 1e9),
                                           of_hbm_peak=round(b / t / HBM_PEAK, 3))
    posb = torch.full((bs,), (ctx // P) * P - 1, device=dev, dtype=torch.int64)       # every sequence completes a block
    t = _timed(lambda: ops.pool_kv_blocks(kc, vc, pk, pv, rtt, rpi, posb, P), 20)
    res["pool_kv_blocks_decode (every sequence ends a block)"] = dict(us=round(t * 1e6, 1), gbs=round(bs * (P + 1) * G * d * 2 * 2 / t / 1e9))
    # ---- prefill attention
    T = prefill_bs * prefill_len
    kp = torch.randn(T + 8, G, d, device=dev, generator=g).to(dt)
    vp = torch.randn(T + 8, G, d, device=dev, generator=g).to(dt)
    pkp, pvp = torch.randn_like(kp), torch.randn_like(vp)
    rtp = (torch.arange(T, device=dev, dtype=torch.int32) + 1).view(prefill_bs, prefill_len)
    qp = torch.randn(T, H, d, device=dev, generator=g).to(dt)
    gp = torch.randn(T, H, device=dev, generator=g).to(dt)
    op = torch.empty_like(qp)
    posp = torch.arange(prefill_len, device=dev).repeat(prefill_bs)
    tok_req = torch.repeat_interleave(torch.arange(prefill_bs, device=dev, dtype=torch.int32), prefill_len)
    rpp = torch.arange(prefill_bs, device=dev)
    bq = ops.window_attention_block_tokens(H, G, d, d, dt)
    assert prefill_len % bq == 0
    starts = torch.arange(0, T, bq, dtype=torch.int32)
    blocks = torch.stack([starts, torch.full_like(starts, bq)], 1).to(dev)
    t = _timed(lambda: ops.window_attention(qp, kp, vp, op, rtp, rpp, posp, sink, W, d ** -0.5, tok_req=tok_req, blocks=blocks, max_run=bq, pool=P,
                                            pooled_k=pkp, pooled_v=pvp, head_gate=gp), 3)
    pairs = prefill_bs * sum(min(i + 1, W) + max(0, (i - W + 1) // P) for i in range(prefill_len))
    fl = pairs * H * 2 * 2 * d
    res["fudonex_prefill_attention"] = dict(ms=round(t * 1e3, 3), tflops=round(fl / t / 1e12, 1), of_mfma_peak=round(fl / t / MFMA_BF16_PEAK, 3))
    t = _timed(lambda: ops.window_attention(qp, kp, vp, op, rtp, rpp, posp, sink, W, d ** -0.5, tok_req=tok_req, blocks=blocks, max_run=bq), 3)
    pairs = prefill_bs * sum(min(i + 1, W) for i in range(prefill_len))
    fl = pairs * H * 2 * 2 * d
    res["gatarax_prefill_attention"] = dict(ms=round(t * 1e3, 3), tflops=round(fl / t / 1e12, 1), of_mfma_peak=round(fl / t / MFMA_BF16_PEAK, 3))
    t = _timed(lambda: ops.pool_kv_blocks(kp, vp, pkp, pvp, rtp, rpp, posp, P, tok_req=tok_req), 5)
    res["pool_kv_blocks_prefill"] = dict(us=round(t * 1e6, 1), gbs=round(T * (1 + 1.0 / P) * G * d * 2 * 2 / t / 1e9))
    # ---- the recurrences
    RH, RG, dk, dv, MG = s["rec_heads"], s["rec_kv_heads"], s["rec_dim"], s["rec_vdim"], s["groups"]
    state = torch.zeros(bs + 1, RH, dk, dv, device=dev)
    r2s = torch.arange(1, bs + 1, device=dev, dtype=torch.int32)
    zeros_h = torch.zeros(RH, device=dev)
    ones_h = torch.ones(RH, device=dev)
    decay = torch.full((RH,), 0.97, device=dev)
    rb_c = torch.zeros(RH * dk, device=dev)
    ss = torch.arange(0, T, prefill_len, device=dev, dtype=torch.int32)
    sl = torch.full((prefill_bs,), prefill_len, device=dev, dtype=torch.int32)
    for n, seg, reps in ((bs, {}, 20), (T, dict(tok_req=tok_req, seg_start=ss, seg_len=sl), 3)):
        rp_, ps_ = (rpi, torch.full((bs,), ctx, device=dev, dtype=torch.int64)) if not seg else (rpp, posp)
        xs = torch.randn(n, RH, dv, device=dev, generator=g).to(dt)
        Bm, Cm = (torch.randn(n, MG, dk, device=dev, generator=g).to(dt) * 0.1 for _ in range(2))
        dtl = torch.randn(n, RH, device=dev, generator=g)
        od = torch.empty(n, RH, dv, device=dev)
        t = _timed(lambda: ops.linear_recurrence(Cm, Bm, xs, od, state, r2s, rp_, ps_, 1.0, dt_logits=dtl, dt_bias=zeros_h, rate_log=zeros_h,
                                                 skip=ones_h, **seg), reps)
        qg, kg = (torch.randn(n, RH, dk, device=dev, generator=g).to(dt) * 0.1 for _ in range(2))
        t2 = _timed(lambda: ops.linear_recurrence(qg, kg, xs, od, state, r2s, rp_, ps_, 1.0, head_decay=decay, **seg), reps)
        qd = torch.nn.functional.normalize(torch.randn(n, RG, dk, device=dev, generator=g), dim=-1)
        kd = torch.nn.functional.normalize(torch.randn(n, RG, dk, device=dev, generator=g), dim=-1)
        ba = torch.randn(n, 2 * RH, device=dev, generator=g)
        t3 = _timed(lambda: ops.gated_delta_rule(qd, kd, xs, ba[:, :RH], ba[:, RH:], zeros_h, zeros_h, od, state, r2s, rp_, ps_, dk ** -0.5, **seg), reps)
        be = torch.randn(n, RH, device=dev, generator=g).to(dt)
        z = torch.randn(n, RH * dk, device=dev, generator=g)
        t4 = _timed(lambda: ops.gated_delta_rule(qd, kd, xs, be, z, rb_c, zeros_h, od, state, r2s, rp_, ps_, dk ** -0.5, **seg), reps)
        state.zero_()
        if not seg:
            b = bs * RH * dk * dv * 4 * 2
            for name, tt in (("fudonex_state_space_decode", t), ("gatarax_lightning_decode", t2), ("fudonex_delta_rule_decode", t3),
                             ("gatarax_delta_rule_decode", t4)):
                res[name] = dict(us=round(tt * 1e6, 1), gbs=round(b / tt / 1e9), of_hbm_peak=round(b / tt / HBM_PEAK, 3))
        else:
            for name, tt, fl_ in (("fudonex_state_space_prefill", t, 6), ("gatarax_lightning_prefill", t2, 6), ("fudonex_delta_rule_prefill", t3, 10),
                                  ("gatarax_delta_rule_prefill", t4, 10)):
                res[name] = dict(ms=round(tt * 1e3, 3), vector_tflops=round(T * RH * dk * dv * fl_ / tt / 1e12, 2),
                                 tokens_per_s_per_sequence=round(prefill_len / tt))
    return res


def fudonex_stream_kernels(s: dict, tokens: int, segments: int) -> dict:
    """The elementwise launches by bytes moved (bf16 activations, fp32 stream), each beside the closest model's like launch."""
    from . import ops
    from .layers.rotary_embedding import pair_inv_freq, scaled_pair_inv_freq

    dev, dt = "cuda", torch.bfloat16
    D = s["width"]
    g = torch.Generator(device=dev).manual_seed(0)
    res = {}
    x = torch.randn(tokens, D, device=dev, generator=g)
    y = torch.randn(tokens, D, device=dev, generator=g).to(dt)
    w = torch.zeros(D, device=dev, dtype=dt)
    ls = torch.ones(D, device=dev, dtype=dt)
    t = _timed(lambda: ops.rmsnorm_residual_add(x, y, w, 1e-6, offset=1.0, layer_scale=ls, mult=0.5), 20)
    res["rmsnorm_residual_add (offset weight, layer scale)"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * D * (4 + 4 + 2 + 2) / t / 1e9))
    t = _timed(lambda: ops.branch_residual_add(x, y, ls, eps=1e-6), 20)
    res["branch_residual_add, one normed branch (closest)"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * D * (4 + 4 + 2) / t / 1e9))
    t = _timed(lambda: ops.offset_rmsnorm(x, w, 1e-6, 1.0), 20)
    res["offset_rmsnorm (closest, the norm in front of a sublayer)"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * D * (4 + 2) / t / 1e9))
    # gate, then group norm  |  head norm, then gate
    RH, dv = s["rec_heads"], s["rec_vdim"]
    inner = RH * dv
    yv = torch.randn(tokens, inner, device=dev, generator=g)
    z = torch.randn(tokens, inner, device=dev, generator=g).to(dt)
    wi = torch.ones(inner, device=dev, dtype=dt)
    t = _timed(lambda: ops.gated_group_rmsnorm(yv, z, wi, s["norm_groups"], 1e-6), 20)
    res["gated_group_rmsnorm"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * inner * (4 + 2 + 2) / t / 1e9))
    wv = torch.ones(dv, device=dev, dtype=dt)
    t = _timed(lambda: ops.head_rmsnorm_gate_act(yv.view(tokens, RH, dv), wv, z, 1e-6, dt, "sigmoid"), 20)
    res["head_rmsnorm_gate (closest)"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * inner * (4 + 2 + 2) / t / 1e9))
    # convolution over x | B | C with bias and silu  |  over q | k | v with silu
    C = inner + 2 * s["groups"] * s["rec_dim"]
    taps = s["conv"]
    u = torch.randn(tokens, C + inner, device=dev, generator=g).to(dt)[:, inner:]
    w1 = torch.randn(C, taps, device=dev, generator=g).to(dt)
    bias = torch.randn(C, device=dev, generator=g).to(dt)
    state = torch.zeros(segments + 1, taps - 1, C, device=dev)
    r2s = torch.arange(1, segments + 1, device=dev, dtype=torch.int32)
    rpi = torch.arange(segments, device=dev)
    per = tokens // segments
    if per == 1:
        seg, pos = {}, torch.full((tokens,), 100, device=dev, dtype=torch.int64)
    else:
        seg = dict(tok_req=torch.repeat_interleave(torch.arange(segments, device=dev, dtype=torch.int32), per),
                   seg_start=torch.arange(0, tokens, per, device=dev, dtype=torch.int32),
                   seg_len=torch.full((segments,), per, device=dev, dtype=torch.int32))
        pos = torch.arange(per, device=dev).repeat(segments)
    t = _timed(lambda: ops.causal_conv(u, w1, state, r2s, rpi, pos, act="silu", bias=bias, **seg), 20)
    res["causal_conv (bias, silu; with the state's update)"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * C * 2 * 2 / t / 1e9))
    t = _timed(lambda: ops.causal_conv(u, w1, state, r2s, rpi, pos, act="silu", **seg), 20)
    res["causal_conv (silu; closest)"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * C * 2 * 2 / t / 1e9))
    # head norm + rotation of q (scaled frequencies and magnitude | plain)
    H, d = s["heads"], s["dim"]
    qs = torch.randn(tokens, H * d + 64, device=dev, generator=g).to(dt)[:, : H * d].view(tokens, H, d)
    wq = torch.ones(d, device=dev, dtype=dt)
    f, mag = scaled_pair_inv_freq(10000.0, s["rot"], dict(factor=4.0, original=2048, fast=16.0, slow=2.0))
    f, f0 = f.to(dev), pair_inv_freq(10000.0, s["rot"]).to(dev)
    t = _timed(lambda: ops.head_norm_rope(qs, wq, 1e-6, pos, f, s["rot"], False, 1.0, dt, rot_mag=mag), 20)
    res["head_norm_rope (scaled frequencies, magnitude)"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * H * d * 2 * 2 / t / 1e9))
    t = _timed(lambda: ops.head_norm_rope(qs, wq, 1e-6, pos, f0, s["rot"], False, 1.0, dt), 20)
    res["head_norm_rope (closest)"] = dict(us=round(t * 1e6, 1), gbs=round(tokens * H * d * 2 * 2 / t / 1e9))
    # q, k and v of an attention layer: one launch beside the three it replaces
    G = s["kv_heads"]
    qkv = torch.randn(tokens, (H + 2 * G) * d + 64, device=dev, generator=g).to(dt)
    q_, k_, v_ = qkv[:, : H * d].view(tokens, H, d), qkv[:, H * d: (H + G) * d].view(tokens, G, d), qkv[:, (H + G) * d: (H + 2 * G) * d].view(tokens, G, d)
    kc, vc = torch.zeros(tokens + 8, G, d, device=dev, dtype=dt), torch.zeros(tokens + 8, G, d, device=dev, dtype=dt)
    loc = torch.arange(1, tokens + 1, device=dev)
    byt = tokens * (H + 2 * G) * d * 2 * 2
    t = _timed(lambda: ops.qkv_norm_rope_write(q_, k_, v_, wq, wq, 1e-6, pos, f, s["rot"], False, mag, kc, vc, loc), 20)
    res["qkv_norm_rope_write (one launch)"] = dict(us=round(t * 1e6, 1), gbs=round(byt / t / 1e9))

    def three():
        ops.head_norm_rope(q_, wq, 1e-6, pos, f, s["rot"], False, 1.0, dt, rot_mag=mag)
        ops.head_norm_rope(k_, wq, 1e-6, pos, f, s["rot"], False, 1.0, dt, cache=kc, loc=loc, rot_mag=mag)
        ops.head_norm_rope(v_, wq, 1e-6, pos, f, 0, False, 1.0, dt, cache=vc, loc=loc)
    t = _timed(three, 20)
    res["head_norm_rope x 3 (what it replaces)"] = dict(us=round(t * 1e6, 1), gbs=round(byt / t / 1e9))
    return res


def run_fudonex(size: str, dtype: str = "bfloat16", steps: int = 32, prefill_bs: int = 4, prefill_len: int = 2048, decode_bs: int = 64,
                decode_ctx: int = 1024) -> dict:
    s = FUDONEX_SIZES[size]
    if size == "fxtiny":
        prefill_bs, prefill_len, decode_bs, decode_ctx = 2, 256, 8, 128
    out = dict(size=size, shape=s, dtype=dtype, data="synthetic", workload=dict(prefill=[prefill_bs, prefill_len], decode=[decode_bs, decode_ctx], steps=steps))
    out["fudonex"] = model_throughput(fudonex_config(s), dtype, prefill_bs, prefill_len, decode_bs, decode_ctx, steps, graph=False)
    out["gatarax"] = model_throughput(gatarax_dense_config(s), dtype, prefill_bs, prefill_len, decode_bs, decode_ctx, steps, graph=False)
    out["mixers"] = fudonex_mixer_kernels(s, decode_bs, decode_ctx, prefill_bs, prefill_len)
    out["stream_decode"] = fudonex_stream_kernels(s, decode_bs, decode_bs)
    out["stream_prefill"] = fudonex_stream_kernels(s, prefill_bs * prefill_len, prefill_bs)
    return out
