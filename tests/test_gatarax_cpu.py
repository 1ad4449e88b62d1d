"""Gatarax on the CPU: the package's host side (configuration, weight stacking, model wiring, ScheduleBatch /
ForwardBatch, the KV / request / state pools, TraceReplayer, Scheduler) runs with the CPU stand-in ops (tests/cpu_ops.py)
and every logit is compared with the plain whole-sequence implementation in oracle/gatarax_ref.py.  The HIP kernels
have their own file (test_gatarax_gpu.py); here the arithmetic is the stand-in's, the bookkeeping is the package's."""
import pytest
import torch

import gatarax_cases as cases
import gatarax_util as gu
from oracle import gatarax_ref as ref

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
    cfg = gu.make_config()
    return cfg, gu.make_weights(cfg, seed=3)


def test_oracle_closed_forms_agree_with_their_step_forms():
    """The oracle states the fixed-decay recurrence as an explicit sum over earlier tokens and the sink as an extra term of
    the denominator; stepping the matrix, and a softmax over the scores with a zero appended, give the same."""
    g = torch.Generator().manual_seed(0)
    T, H, d, dv = 13, 2, 5, 4
    q, k, v = (torch.randn(T, H, n, generator=g, dtype=torch.float64) for n in (d, d, dv))
    decay = torch.tensor([0.9, 0.6], dtype=torch.float64)
    S = torch.zeros(H, d, dv, dtype=torch.float64)
    want = ref.decayed_sum(q, k, v, decay)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        assert (torch.einsum("hkv,hk->hv", S, q[t]) - want[t]).abs().max() < 1e-10
    o = ref.window_sink_attention(q, k[:, :1], v[:, :1], 0.7, 4)
    for i in (0, 3, 9):
        lo = max(0, i - 3)
        s = torch.cat([(k[lo:i + 1, 0] @ q[i, 1]) * 0.7, torch.zeros(1, dtype=torch.float64)])
        assert (torch.softmax(s, 0)[:-1] @ v[lo:i + 1, 0] - o[i, 1]).abs().max() < 1e-12


@pytest.mark.parametrize("kind", ["parallel", "lightning"])
@pytest.mark.parametrize("mlp", ["none", "dense", "moe"])
def test_each_mixer_and_feed_forward_alone(kind, mlp):
    """One-layer models: whole, cut, and token by token."""
    mixer = gu.parallel() if kind == "parallel" else gu.lightning()
    ff = dict(none=None, dense=gu.dense(24), moe=gu.moe())[mlp]
    cfg = gu.make_config(layers=[(mixer, ff)])
    w = gu.make_weights(cfg, seed=1)
    prompts = gu.random_prompts(cfg, [19])
    mr = gu.build_runner(cfg, w)
    gu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 19)]], TOL)
    gu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 7)], [("r0", 2)]] + [[("r0", 1)] for _ in range(10)], TOL)
    assert gu.pools_are_whole(mr)


def test_whole_prompt_then_token_by_token(model):
    cfg, w = model
    prompts = gu.random_prompts(cfg, [23])
    mr = gu.build_runner(cfg, w)
    gu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 23)]], TOL)
    gu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 1)] for _ in range(23)], TOL)
    gu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 9)]] + [[("r0", 1)] for _ in range(14)], TOL)
    assert gu.pools_are_whole(mr)


@pytest.mark.parametrize("sizes", [[2, 2, 2, 3, 5, 2, 7, 1, 1, 2], [1, 4, 4, 4, 4, 4, 4, 2], [25, 2]])
def test_portions_of_any_size(model, sizes):
    cfg, w = model
    prompts = gu.random_prompts(cfg, [sum(sizes)], seed=5)
    mr = gu.build_runner(cfg, w)
    gu.replay_and_compare(mr, cfg, w, prompts, [[("r0", k)] for k in sizes], TOL)
    assert gu.pools_are_whole(mr)


@pytest.mark.parametrize("page_size", [1, 4])
def test_mixed_batches_reuse_slots_and_pages(model, page_size):
    """Unequal requests side by side -- portions beside single tokens, a request that sits a step out, requests that end
    while others go on -- in a pool so small that KV slots, request rows and state slots are all handed out again."""
    cfg, w = model
    prompts = gu.random_prompts(cfg, [17, 9, 1, 12, 20, 6], seed=7)
    sched = [[("r0", 5), ("r1", 2)], [("r0", 1), ("r1", 7), ("r2", 1)], [("r0", 4), ("r3", 3)], [("r3", 1)],
             [("r0", 1), ("r3", 1)], [("r0", 6), ("r3", 7), ("r4", 2)], [("r4", 1), ("r5", 1)], [("r4", 1), ("r5", 1)],
             [("r4", 9), ("r5", 4)], [("r4", 1)], [("r4", 6)]]
    mr = gu.build_runner(cfg, w, max_total_tokens=48, max_running_requests=3, page_size=page_size)
    want = {k: ref.forward(gu.public(cfg), w, p) for k, p in prompts.items()}
    gu.replay_and_compare(mr, cfg, w, prompts, sched, TOL, want_all=want)
    assert gu.pools_are_whole(mr)
    # the same again on the used pools: stale keys, stale matrices, stale convolution inputs
    gu.replay_and_compare(mr, cfg, w, prompts, sched, TOL, want_all=want)
    assert gu.pools_are_whole(mr)


def test_equal_and_unit_sizes():
    """Sizes that a model may happen to make equal or 1: one head, as many key heads as query heads, a window of 1 (a token
    sees itself and the sink), convolutions of 2 taps and of as many taps as the input convolution, key and value widths
    equal, one expert group, every group kept, one expert per token, every expert per token, embedding and logit factors of
    1, width equal to the vocabulary, a decay of 1, a layer without feed-forward."""
    layers = [(gu.parallel(heads=2, kv_heads=2, dim=8, vdim=8, window=1, conv=2, r_heads=1, r_kv_heads=1, r_dim=8, r_vdim=8, r_conv=2,
                           decay_rank=1, gate_rank=1), gu.moe(experts=3, top=1, count=1, keep=1, ff=8)),
              (gu.lightning(heads=1, dim=4, vdim=4, decay=(1.0,)), None),
              (gu.parallel(heads=3, kv_heads=1, dim=4, vdim=4, window=3, conv=2, r_heads=3, r_kv_heads=3, r_dim=4, r_vdim=4, r_conv=2),
               gu.moe(experts=4, top=4, count=4, keep=4, ff=4)),
              (gu.lightning(heads=2, dim=8, vdim=8, decay=(0.5, 0.5)), gu.dense(16))]
    cfg = gu.make_config(layers=layers, width=16, vocab=16, taps=2, embed_scale=1.0, logit_scale=1.0)
    w = gu.make_weights(cfg, seed=11)
    prompts = gu.random_prompts(cfg, [14, 5], seed=1)
    mr = gu.build_runner(cfg, w, max_total_tokens=32)
    gu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 3), ("r1", 1)], [("r0", 1), ("r1", 1)], [("r0", 10), ("r1", 3)]], TOL)


def test_state_is_what_the_next_step_reads(model):
    """Cutting a prompt must hand over exactly the layers' matrices and convolution inputs: a corrupted one changes the
    next portion's logits, a sequence's first token reads none of what its slot held, and a finished request's slot goes
    to the next one."""
    cfg, w = model
    from sglang_custom_amd.managers.trace_replay import TraceReplayer

    prompts = gu.random_prompts(cfg, [8], seed=2)["r0"]
    mr = gu.build_runner(cfg, w)
    pool = mr.req_to_token_pool.state_pool
    assert sorted(pool.matrices) == [0, 1, 2, 3] and pool.matrices[1].shape[1:] == (3, 8, 12)
    assert pool.convs[(0, "canon")].shape[1:] == (2, 48) and pool.convs[(2, "left")].shape[1:] == (1, 2 * 8 + 8 + 16)
    assert pool.convs[(0, "right")].shape[1:] == (3, 2 * 2 * 8 + 4 * 12) and (1, "left") not in pool.convs
    for m in list(pool.matrices.values()) + list(pool.convs.values()):
        m.fill_(123.0)
    rp = TraceReplayer(mr)
    want = ref.forward(gu.public(cfg), w, prompts)
    assert gu.rel_err(rp.step([dict(id="a", tokens=prompts[:4], want=[0, 1, 2, 3])]), want[:4]) < TOL
    slot = rp.live["a"].state_slot
    for kind, key in (("matrices", 2), ("convs", (3, "canon")), ("convs", (0, "left")), ("convs", (2, "right"))):
        good = {k: t[slot].clone() for k, t in list(pool.matrices.items()) + list(pool.convs.items())}
        getattr(pool, kind)[key][slot] += 0.5
        assert gu.rel_err(rp.step([dict(id="a", tokens=prompts[4:5], want=[0])]), want[4:5]) > 1e-4, (kind, key)
        rp.finish("a")
        rp.step([dict(id="a", tokens=prompts[:4], want=[])])
        slot = rp.live["a"].state_slot
        for k, t in list(pool.matrices.items()) + list(pool.convs.items()):
            assert torch.equal(t[slot], good[k]), k
    assert gu.rel_err(rp.step([dict(id="a", tokens=prompts[4:], want=[0, 1, 2, 3])], ["a"]), want[4:]) < TOL
    assert gu.pools_are_whole(mr)


@pytest.mark.parametrize("chunk,mixed", [(None, False), (6, False), (6, True)])
def test_greedy_generation_through_the_scheduler(model, chunk, mixed):
    """The package's own entry point: requests queued at the Scheduler, prompts chunked by its policy, decode batches
    (and decode tokens riding prefill batches) formed by it, tokens picked by the Sampler."""
    from sglang_custom_amd.managers.schedule_batch import Req
    from sglang_custom_amd.managers.scheduler import Scheduler
    from sglang_custom_amd.sampling.sampling_params import SamplingParams

    cfg, w = model
    prompts = gu.random_prompts(cfg, [11, 3, 7, 15, 1], seed=9)
    mr = gu.build_runner(cfg, w, max_total_tokens=96, max_running_requests=3, chunked_prefill_size=chunk, enable_mixed_chunk=mixed)
    sch = Scheduler(mr)
    for k, p in prompts.items():
        sch.add_request(Req(k, p, SamplingParams(temperature=0, max_new_tokens=6)))
    done = sch.run_until_done()
    for k, p in prompts.items():
        assert done[k].output_ids == ref.greedy(gu.public(cfg), w, p, 6), k
    assert gu.pools_are_whole(mr)
    if chunk:
        assert sch.num_prefill_batches > 3


def test_prefix_cache_is_refused(model):
    from sglang_custom_amd.managers.scheduler import Scheduler

    cfg, w = model
    with pytest.raises(ValueError):
        Scheduler(gu.build_runner(cfg, w), enable_radix_cache=True)


def test_configuration_is_read_not_assumed():
    from sglang_custom_amd.configs.model_config import ModelConfig
    from sglang_custom_amd.models.registry import get_model_class

    cfg = gu.public(gu.make_config())
    mc = ModelConfig(cfg, dtype="float32")
    assert mc.architecture == "Gatarax" and get_model_class(mc.architecture).__name__ == "GataraxForCausalLM"
    assert mc.kv_layer_shapes == [(2, 16, 8), None, (1, 8, 16), None]
    assert mc.recurrent_layer_shapes == [(4, 8, 12), (3, 8, 12), (2, 12, 4), (1, 20, 4)]
    assert mc.canon_taps == 3 and mc.embedding_scale == 3.0 and mc.logit_scale == 0.5 and mc.rms_norm_eps == 1e-5
    bad = gu.public(gu.make_config())
    bad["layers"][1]["type"] = "something_else"
    with pytest.raises(ValueError):
        ModelConfig(bad)
    bad = gu.public(gu.make_config())
    bad["layers"][1]["mixer"]["decay"] = [0.5]
    with pytest.raises(ValueError):
        ModelConfig(bad)
    bad = gu.public(gu.make_config())
    bad["layers"][0]["mlp"]["kind"] = "other"
    with pytest.raises(ValueError):
        ModelConfig(bad)


# ---- the stand-in ops themselves against the oracle's functions: the same cases the HIP kernels run on the GPU
def test_standins_norms_gates_convolutions():
    import cpu_ops

    cases.check_offset_norm_and_branch_add(cpu_ops, "cpu", torch.float32)
    cases.check_gates_and_activations(cpu_ops, "cpu", torch.float32)
    cases.check_conv(cpu_ops, "cpu", torch.float32, taps=4, cuts=(20, 2, 1, 14), two=True, residual=True)
    cases.check_conv(cpu_ops, "cpu", torch.float32, taps=3, cuts=(1, 1, 33, 1, 1), act="silu", decode_tail=2)
    cases.check_conv(cpu_ops, "cpu", torch.float32, taps=2, T=1, cuts=(1,))
    cases.check_conv_planted(cpu_ops, "cpu", torch.float32)
    cases.check_conv_batch(cpu_ops, "cpu", torch.float32)


def test_standins_attention_delta_rule_mixture():
    import cpu_ops

    cases.check_window_attention(cpu_ops, "cpu", torch.float32, T=40, window=7, cuts=(17, 2, 20, 1), decode_tail=1)
    cases.check_window_attention(cpu_ops, "cpu", torch.float32, T=30, window=1, dv=8, cuts=(30,))
    cases.check_delta_rule(cpu_ops, "cpu", torch.float32, cuts=(20, 2, 1, 22))
    cases.check_delta_rule(cpu_ops, "cpu", torch.float32, cuts=(3, 40, 1, 1), decode_tail=2)
    cases.check_router_softmax(cpu_ops, "cpu")
    cases.check_router_softmax(cpu_ops, "cpu", E=8, n_groups=8, keep=3, top=2)
    cases.check_gated_experts(cpu_ops, "cpu", torch.float32)
