"""Fudonex on the CPU: the package's host side (configuration, weight stacking, model wiring, ScheduleBatch /
ForwardBatch, the KV / request / state pools with averaged blocks and borrowed caches, TraceReplayer, Scheduler) runs with
the CPU stand-in ops (tests/cpu_ops.py) and every logit is compared with the plain whole-sequence implementation in
oracle/fudonex_ref.py.  The HIP kernels have their own file (test_fudonex_gpu.py); here the arithmetic is the stand-in's,
the bookkeeping is the package's."""
import pytest
import torch

import fudonex_cases as cases
import fudonex_util as fu
from oracle import fudonex_ref as ref

TOL = 2e-5


@pytest.fixture(autouse=True)
def _cpu_backend():
    import cpu_ops
    from sglang_custom_amd import ops_backend
    from sglang_custom_amd.distributed import parallel_state

    prev = ops_backend._backend
    ops_backend.set_ops_backend(cpu_ops)
    parallel_state.init_distributed_environment(1, 0)
    yield
    ops_backend.set_ops_backend(prev)


@pytest.fixture(scope="module")
def model():
    cfg = fu.make_config()
    return cfg, fu.make_weights(cfg, seed=3)


def test_oracle_restatements_agree():
    """The oracle's attention against a second statement of it: explicit lists of what a token sees, a softmax over the
    scores with the sink appended."""
    g = torch.Generator().manual_seed(0)
    T, H, d, dv, W, P = 23, 2, 5, 4, 6, 4
    q, k, v = (torch.randn(T, n, m, generator=g, dtype=torch.float64) for n, m in ((H, d), (1, d), (1, dv)))
    sink = torch.tensor([0.3, -1.0], dtype=torch.float64)
    o = ref.pooled_window_attention(q, k, v, 0.7, W, P, sink)
    for i in (0, 5, 6, 9, 10, 13, 22):
        toks = [j for j in range(T) if 0 <= i - j < W]
        blks = [b for b in range(T // P) if b * P + P - 1 <= i - W]
        assert len(blks) == max(0, (i - W + 1) // P)
        keys = torch.stack([k[b * P:(b + 1) * P, 0].mean(0) for b in blks] + [k[j, 0] for j in toks])
        vals = torch.stack([v[b * P:(b + 1) * P, 0].mean(0) for b in blks] + [v[j, 0] for j in toks])
        s = torch.cat([(keys @ q[i, 1]) * 0.7, sink[1:2]])
        assert (torch.softmax(s, 0)[:-1] @ vals - o[i, 1]).abs().max() < 1e-12
    # token 13 (window 8..13) sees blocks 0 and 1; token 12 (window 7..12) sees block 0 alone, and tokens 4..6 not at all
    assert [b for b in range(T // P) if b * P + P - 1 <= 13 - W] == [0, 1] and [b for b in range(T // P) if b * P + P - 1 <= 12 - W] == [0]


@pytest.mark.parametrize("kind", ["attention", "mamba2", "delta"])
@pytest.mark.parametrize("mlp", ["none", "dense"])
def test_each_mixer_alone(kind, mlp):
    """One-layer models: whole, cut, and token by token."""
    mixer = dict(attention=fu.attention(), mamba2=fu.mamba2(), delta=fu.delta())[kind]
    cfg = fu.make_config(layers=[(mixer, None if mlp == "none" else fu.dense(24))])
    w = fu.make_weights(cfg, seed=1)
    prompts = fu.random_prompts(cfg, [25])
    mr = fu.build_runner(cfg, w)
    fu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 25)]], TOL)
    fu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 7)], [("r0", 2)]] + [[("r0", 1)] for _ in range(16)], TOL)
    assert fu.pools_are_whole(mr)


def test_whole_prompt_then_token_by_token(model):
    cfg, w = model
    prompts = fu.random_prompts(cfg, [31])
    mr = fu.build_runner(cfg, w)
    fu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 31)]], TOL)
    fu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 1)] for _ in range(31)], TOL)
    fu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 9)]] + [[("r0", 1)] for _ in range(22)], TOL)
    assert fu.pools_are_whole(mr)


@pytest.mark.parametrize("sizes", [[2, 2, 2, 3, 5, 2, 7, 1, 1, 2, 6], [1, 4, 4, 4, 4, 4, 4, 2, 3, 3], [31, 2]])
def test_portions_of_any_size(model, sizes):
    cfg, w = model
    prompts = fu.random_prompts(cfg, [sum(sizes)], seed=5)
    mr = fu.build_runner(cfg, w)
    fu.replay_and_compare(mr, cfg, w, prompts, [[("r0", k)] for k in sizes], TOL)
    assert fu.pools_are_whole(mr)


@pytest.mark.parametrize("page_size", [1, 4, 6])
def test_mixed_batches_reuse_slots_and_pages(model, page_size):
    """Unequal requests side by side -- portions beside single tokens, a request that sits a step out, requests that end
    while others go on -- in a pool so small that KV slots, averaged rows, request rows and state slots are all handed out
    again.  Layer 0 keeps averages over blocks of 3 (its own) and of 2 (for the layer that reads its cache).  Pages of 6 hold
    whole blocks of 3 and of 2 (one averaged row per block of slots), pages of 4 hold whole blocks of 2 only, single-slot pages
    none."""
    cfg, w = model
    prompts = fu.random_prompts(cfg, [27, 9, 1, 12, 30, 6], seed=7)
    sched = [[("r0", 5), ("r1", 2)], [("r0", 1), ("r1", 7), ("r2", 1)], [("r0", 4), ("r3", 3)], [("r3", 1)],
             [("r0", 1), ("r3", 1)], [("r0", 16), ("r3", 7), ("r4", 2)], [("r4", 1), ("r5", 1)], [("r4", 1), ("r5", 1)],
             [("r4", 19), ("r5", 4)], [("r4", 1)], [("r4", 6)]]
    mr = fu.build_runner(cfg, w, max_total_tokens=72, max_running_requests=3, page_size=page_size)
    divs = {l: d for l, (_, _, d) in mr.token_to_kv_pool.pooled.items()}
    assert divs == {(0, 3): 3 if page_size == 6 else 1, (0, 2): 2 if page_size != 1 else 1, (4, 2): 2 if page_size != 1 else 1}
    want = {k: ref.forward(cfg, w, p) for k, p in prompts.items()}
    fu.replay_and_compare(mr, cfg, w, prompts, sched, TOL, want_all=want)
    assert fu.pools_are_whole(mr)
    # the same again on the used pools: stale keys, stale averages, stale matrices, stale convolution inputs
    fu.replay_and_compare(mr, cfg, w, prompts, sched, TOL, want_all=want)
    assert fu.pools_are_whole(mr)


def test_equal_and_unit_sizes():
    """Sizes that a model may happen to make equal or 1: one head, as many key heads as query heads, a window of 1 and
    blocks of 1 (every earlier token is its own block), blocks as long as the window, the whole head rotated, no rotation, no
    frequency scaling, one group, as many groups as heads, one norm part, convolutions of 2 taps, key and value widths equal,
    embedding factor, stream factor of 1, no cap on the logits, width equal to the vocabulary, layers without feed-forward."""
    layers = [(fu.attention(heads=2, kv_heads=2, dim=8, vdim=8, window=1, pool=1, rot_dims=8, scaling=False), fu.dense(8)),
              (fu.mamba2(heads=1, vdim=4, state=4, groups=1, norm_groups=1, conv=2), None),
              (fu.delta(heads=1, kv_heads=1, dim=8, vdim=8, conv=2), None),
              (fu.attention(heads=3, kv_heads=1, dim=4, vdim=4, window=3, pool=3, rot_dims=0), fu.dense(16)),
              (fu.mamba2(heads=2, vdim=8, state=8, groups=2, norm_groups=16, conv=2), fu.dense(16)),
              (fu.attention(heads=2, kv_heads=2, dim=8, vdim=8, window=1, pool=1, rot_dims=8, scaling=False, kv_from=0), None),
              (fu.delta(heads=3, kv_heads=3, dim=4, vdim=4, conv=4), fu.dense(4))]
    cfg = fu.make_config(layers=layers, width=16, vocab=16, embed_scale=1.0, residual_mult=1.0, softcap=None)
    w = fu.make_weights(cfg, seed=11)
    prompts = fu.random_prompts(cfg, [14, 5], seed=1)
    mr = fu.build_runner(cfg, w, max_total_tokens=32)
    fu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 3), ("r1", 1)], [("r0", 1), ("r1", 1)], [("r0", 10), ("r1", 3)]], TOL)


def test_attention_only_model_keeps_no_state():
    cfg = fu.make_config(layers=[(fu.attention(), fu.dense()), (fu.attention(kv_from=0), None)])
    w = fu.make_weights(cfg, seed=2)
    mr = fu.build_runner(cfg, w)
    assert mr.req_to_token_pool.state_pool is None
    prompts = fu.random_prompts(cfg, [20, 7], seed=3)
    fu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 6), ("r1", 7)], [("r0", 13)], [("r0", 1)]], TOL)


def test_state_is_what_the_next_step_reads(model):
    """Cutting a prompt must hand over exactly the layers' matrices, convolution inputs and averaged rows: a corrupted one
    changes the next portion's logits; a borrowed cache has no buffers of its own."""
    cfg, w = model
    from sglang_custom_amd.managers.trace_replay import TraceReplayer

    prompts = fu.random_prompts(cfg, [16], seed=2)["r0"]
    mr = fu.build_runner(cfg, w)
    pool, kvp = mr.req_to_token_pool.state_pool, mr.token_to_kv_pool
    assert sorted(pool.matrices) == [1, 2, 5] and pool.matrices[1].shape[1:] == (4, 10, 6) and pool.matrices[2].shape[1:] == (4, 12, 10)
    assert pool.convs[(1, "ssm")].shape[1:] == (2, 4 * 6 + 2 * 2 * 10) and pool.convs[(2, "delta")].shape[1:] == (3, 2 * 2 * 12 + 4 * 10)
    assert kvp.k_buffer[3] is None and kvp.get_key_buffer(3) is kvp.k_buffer[0] and sorted(kvp.pooled) == [(0, 2), (0, 3), (4, 2)]
    for m in list(pool.matrices.values()) + list(pool.convs.values()):
        m.fill_(123.0)
    want = ref.forward(cfg, w, prompts)
    rp = TraceReplayer(mr)
    assert fu.rel_err(rp.step([dict(id="a", tokens=prompts[:12], want=list(range(12)))]), want[:12]) < TOL
    slot = rp.live["a"].state_slot
    bad = []
    for kind, key in (("matrices", 1), ("matrices", 2), ("convs", (1, "ssm")), ("convs", (2, "delta")), ("pooled", (0, 3)), ("pooled", (0, 2))):
        rp2 = TraceReplayer(mr)
        rp2.step([dict(id="b", tokens=prompts[:12], want=[])])
        s2 = rp2.live["b"].state_slot
        if kind == "pooled":
            saved = kvp.pooled[key][0].clone()
            kvp.pooled[key][0].add_(0.5)          # every averaged key of a layer (the blocks token 12 sees among them)
        else:
            getattr(pool, kind)[key][s2] += 0.5
        bad.append(fu.rel_err(rp2.step([dict(id="b", tokens=prompts[12:13], want=[0])], ["b"]), want[12:13]))
        if kind == "pooled":
            kvp.pooled[key][0].copy_(saved)
    assert min(bad) > 1e-4, bad
    assert fu.rel_err(rp.step([dict(id="a", tokens=prompts[12:], want=[0, 1, 2, 3])], ["a"]), want[12:]) < TOL
    assert slot is not None and fu.pools_are_whole(mr)


@pytest.mark.parametrize("chunk,mixed", [(None, False), (6, False), (6, True)])
def test_greedy_generation_through_the_scheduler(model, chunk, mixed):
    """The package's own entry point: requests queued at the Scheduler, prompts chunked by its policy, decode batches
    (and decode tokens riding prefill batches) formed by it, tokens picked by the Sampler."""
    from sglang_custom_amd.managers.schedule_batch import Req
    from sglang_custom_amd.managers.scheduler import Scheduler
    from sglang_custom_amd.sampling.sampling_params import SamplingParams

    cfg, w = model
    prompts = fu.random_prompts(cfg, [11, 3, 7, 15, 1], seed=9)
    mr = fu.build_runner(cfg, w, max_total_tokens=96, max_running_requests=3, chunked_prefill_size=chunk, enable_mixed_chunk=mixed)
    sch = Scheduler(mr)
    for k, p in prompts.items():
        sch.add_request(Req(k, p, SamplingParams(temperature=0, max_new_tokens=6)))
    done = sch.run_until_done()
    for k, p in prompts.items():
        assert done[k].output_ids == ref.greedy(cfg, w, p, 6), k
    assert fu.pools_are_whole(mr)
    if chunk:
        assert sch.num_prefill_batches > 3


def test_prefix_cache_is_refused(model):
    from sglang_custom_amd.managers.scheduler import Scheduler

    cfg, w = model
    with pytest.raises(ValueError):
        Scheduler(fu.build_runner(cfg, w), enable_radix_cache=True)


def test_configuration_is_read_not_assumed():
    from sglang_custom_amd.configs.model_config import ModelConfig
    from sglang_custom_amd.models.registry import get_model_class

    cfg = fu.make_config()
    mc = ModelConfig(cfg, dtype="float32")
    assert mc.architecture == "Fudonex" and get_model_class(mc.architecture).__name__ == "FudonexForCausalLM"
    assert mc.kv_layer_shapes == [(2, 16, 8), None, None, None, (1, 12, 20), None]
    assert mc.kv_layer_sources == {3: 0} and mc.kv_layer_pools == [(2, 3), (), (), (), (2,), ()]
    assert mc.recurrent_layer_shapes == [None, (4, 10, 6), (4, 12, 10), None, None, (3, 5, 8)]
    assert mc.embedding_scale == 2.0 and mc.residual_mult == 0.6 and mc.final_logit_softcapping == 12.0 and mc.rms_norm_eps == 1e-5
    for path, value in ((("layers", 1, "type"), "something_else"), (("layers", 0, "mlp", "kind"), "other"),
                        (("layers", 3, "mixer", "kv_from"), 1), (("layers", 3, "mixer", "kv_from"), 4),
                        (("layers", 3, "mixer", "dim"), 8), (("layers", 3, "mixer", "vdim"), 16),
                        (("layers", 0, "mixer", "rot", "dims"), 7), (("layers", 1, "mixer", "groups"), 3)):
        bad = fu.make_config()
        node = bad
        for k in path[:-1]:
            node = node[k]
        node[path[-1]] = value
        with pytest.raises(ValueError):
            ModelConfig(bad)


# ---- the stand-in ops themselves against the oracle's functions: the same cases the HIP kernels run on the GPU
def test_standins_norms_rotation_convolution():
    import cpu_ops

    cases.check_output_norm_add(cpu_ops, "cpu", torch.float32)
    cases.check_gated_group_norm(cpu_ops, "cpu", torch.float32)
    cases.check_scaled_frequencies()
    cases.check_scaled_rotation(cpu_ops, "cpu", torch.float32)
    cases.check_qkv_norms_one_launch(cpu_ops, "cpu", torch.float32)
    cases.check_conv_bias(cpu_ops, "cpu", torch.float32)


def test_standins_recurrences():
    import cpu_ops

    cases.check_state_space(cpu_ops, "cpu", torch.float32, cuts=(20, 2, 1, 22))
    cases.check_state_space(cpu_ops, "cpu", torch.float32, cuts=(3, 40, 1, 1), decode_tail=2, with_skip=False)
    cases.check_state_space_planted(cpu_ops, "cpu", torch.float32)
    cases.check_delta_rule(cpu_ops, "cpu", torch.float32, cuts=(20, 2, 1, 22))
    cases.check_delta_rule(cpu_ops, "cpu", torch.float32, cuts=(3, 40, 1, 1), decode_tail=2)
    cases.check_delta_rule_planted(cpu_ops, "cpu", torch.float32)


def test_standins_attention_with_averaged_blocks():
    import cpu_ops

    cases.check_pooled_attention(cpu_ops, "cpu", torch.float32, T=60, window=7, pool=4, cuts=(17, 2, 40, 1), decode_tail=1)
    cases.check_pooled_attention(cpu_ops, "cpu", torch.float32, T=50, window=5, pool=4, dv=8, cuts=(50,), page=8)
    cases.check_pooled_attention(cpu_ops, "cpu", torch.float32, T=50, window=9, pool=3, d=20, cuts=(25, 25), page=4, with_gate=False)
    cases.check_pooled_attention_planted(cpu_ops, "cpu", torch.float32, d=8, W=6, P=4)
    cases.check_pooled_attention_planted(cpu_ops, "cpu", torch.float32, d=8, W=6, P=4, page=8)
