"""Gatarax on the GPU: every HIP kernel of the family against the plain functions of oracle/gatarax_ref.py
(gatarax_cases.py holds the cases), then the whole engine (ModelRunner, pools, TraceReplayer, Scheduler) in fp32 and bf16
against the whole-sequence oracle.  Where random numbers would hide a fault -- a key at the window's edge and the one just
past it, a page's border, a value written 600 tokens back, the sink's share, the first tokens of a sequence, stale state in
a reused slot -- the inputs are built so that it shows."""
import pytest
import torch

import gatarax_cases as cases
import gatarax_util as gu
from oracle import gatarax_ref as ref

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(autouse=True)
def _product_ops():
    from sglang_custom_amd import ops_backend
    from sglang_custom_amd.distributed import parallel_state

    ops_backend.set_ops_backend(None)      # the HIP library (get_ops() loads it and raises if it is missing)
    parallel_state.init_distributed_environment(1, 0)
    yield


def ops():
    from sglang_custom_amd.ops_backend import get_ops

    return get_ops()


# ---------------------------------------------------------------------------------------------- kernels, one by one
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D", [48, 40, 1024, 33])
def test_offset_norm_and_branch_sum(dtype, D):
    cases.check_offset_norm_and_branch_add(ops(), DEV, dtype, D=D)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gates_and_activations(dtype):
    cases.check_gates_and_activations(ops(), DEV, dtype)
    cases.check_gates_and_activations(ops(), DEV, dtype, H=1, dv=128)
    cases.check_gates_and_activations(ops(), DEV, dtype, H=6, dv=64)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps,C", [(4, 40), (3, 256), (2, 7), (8, 300), (1, 16)])
def test_short_convolution_whole_cut_and_decoded(dtype, taps, C):
    for cuts, tail in (((37,), 0), ((20, 2, 1, 14), 0), ((17, 16, 2) + (1,) * 2, 2), ((1,) * 37, 37), ((1, 1, 2, 33), 0)):
        cases.check_conv(ops(), DEV, dtype, taps=taps, C=C, cuts=cuts, decode_tail=tail)
    cases.check_conv(ops(), DEV, dtype, taps=taps, C=C, cuts=(5, 2, 30), two=True, residual=True)
    cases.check_conv(ops(), DEV, dtype, taps=taps, C=C, cuts=(36, 1), act="silu", decode_tail=1)
    cases.check_conv(ops(), DEV, dtype, taps=taps, C=C, T=1, cuts=(1,))
    cases.check_conv(ops(), DEV, dtype, taps=taps, C=C, T=2, cuts=(1, 1), decode_tail=1)


@pytest.mark.parametrize("dtype", DTYPES)
def test_short_convolution_edges_first_tokens_and_batches(dtype):
    cases.check_conv_planted(ops(), DEV, dtype)
    cases.check_conv_batch(ops(), DEV, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,d,dv", [(4, 2, 32, 32), (8, 1, 64, 64), (3, 3, 24, 40), (32, 1, 32, 16), (6, 2, 128, 64), (1, 1, 8, 8),
                                      (4, 2, 96, 32), (6, 6, 64, 64), (2, 1, 160, 256), (5, 5, 64, 128)])
def test_window_attention_whole_cut_and_decoded(dtype, H, G, d, dv):
    for window in (40, 1, 33, 500):
        cases.check_window_attention(ops(), DEV, dtype, H=H, G=G, d=d, dv=dv, window=window)
    cases.check_window_attention(ops(), DEV, dtype, H=H, G=G, d=d, dv=dv, window=70, cuts=(60, 3, 2, 85))
    cases.check_window_attention(ops(), DEV, dtype, H=H, G=G, d=d, dv=dv, window=64, cuts=(100,) + (1,) * 50, decode_tail=50, page=16)
    # decode steps whose keys are cut into ranges that a second launch merges: more ranges than tiles, ranges past the window
    cases.check_window_attention(ops(), DEV, dtype, H=H, G=G, d=d, dv=dv, window=500, cuts=(100,) + (1,) * 50, decode_tail=50, splits=3)
    cases.check_window_attention(ops(), DEV, dtype, H=H, G=G, d=d, dv=dv, window=40, cuts=(120,) + (1,) * 30, decode_tail=30, splits=8, page=16)
    cases.check_window_attention(ops(), DEV, dtype, H=H, G=G, d=d, dv=dv, window=20, cuts=(1, 1, 2, 146), pad_q=8)
    cases.check_window_attention(ops(), DEV, dtype, H=H, G=G, d=d, dv=dv, window=9, cuts=(150,), pad_q=3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_window_attention_edges_far_keys_and_the_sink(dtype):
    cases.check_window_attention_planted(ops(), DEV, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,dk,dv", [(4, 2, 12, 20), (4, 4, 32, 32), (2, 2, 32, 64), (2, 1, 64, 64), (1, 1, 128, 96), (6, 3, 200, 33), (1, 1, 1, 1)])
def test_delta_rule_whole_cut_and_decoded(dtype, H, G, dk, dv):
    for cuts, tail in (((45,), 0), ((20, 2, 1, 22), 0), ((17, 16, 2) + (1,) * 10, 10), ((1,) * 45, 45)):
        cases.check_delta_rule(ops(), DEV, dtype, H=H, G=G, dk=dk, dv=dv, cuts=cuts, decode_tail=tail)


@pytest.mark.parametrize("dtype", DTYPES)
def test_delta_rule_far_writes_overwrites_first_tokens_and_slots(dtype):
    cases.check_delta_rule_planted(ops(), DEV, dtype)


def test_router_softmax_groups_by_their_best():
    cases.check_router_softmax(ops(), DEV)
    cases.check_router_softmax(ops(), DEV, E=8, n_groups=8, keep=3, top=2)
    cases.check_router_softmax(ops(), DEV, E=16, n_groups=2, keep=1, top=2, T=300)
    cases.check_router_softmax(ops(), DEV, E=5, n_groups=1, keep=1, top=5)
    cases.check_router_softmax(ops(), DEV, E=128, n_groups=4, keep=2, top=8)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,D,ff,E,top", [(37, 48, 40, 5, 2), (300, 64, 96, 8, 4), (1, 32, 8, 3, 1), (70, 50, 36, 4, 3)])
def test_gated_experts_over_sorted_blocks(dtype, T, D, ff, E, top):
    cases.check_gated_experts(ops(), DEV, dtype, T=T, D=D, ff=ff, E=E, top=top)


def test_gated_experts_over_wide_and_tiled_blocks():
    """Enough rows per expert for the 128-row blocks, and for the 256-row blocks of the prefill projection kernel."""
    cases.check_gated_experts(ops(), DEV, torch.bfloat16, T=1100, D=64, ff=96, E=4, top=2, wide_ok=True, block=128)
    cases.check_gated_experts(ops(), DEV, torch.bfloat16, T=2300, D=128, ff=128, E=4, top=2, tiled_ok=True, block=256)


# ---------------------------------------------------------------------------------------------- the engine
CASES = [("float32", 3e-5), ("bfloat16", 6e-2)]


def _model(dtype, **kw):
    cfg = gu.make_config(layers=gu.default_layers(every_expert=dtype != "float32"), **kw)
    return cfg, gu.make_weights(cfg, seed=3)


@pytest.mark.parametrize("dtype,tol", CASES)
@pytest.mark.parametrize("kind", ["parallel", "lightning"])
def test_each_mixer_alone(dtype, tol, kind):
    mixer = gu.parallel() if kind == "parallel" else gu.lightning()
    cfg = gu.make_config(layers=[(mixer, None)])
    w = gu.make_weights(cfg, seed=1)
    prompts = gu.random_prompts(cfg, [90])
    mr = gu.build_runner(cfg, w, dtype=dtype, device=DEV)
    gu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 90)]], tol)
    gu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 66)], [("r0", 2)]] + [[("r0", 1)] for _ in range(22)], tol)
    assert gu.pools_are_whole(mr)


@pytest.mark.parametrize("dtype,tol", CASES)
def test_prefill_decode_portions_and_batches_against_the_oracle(dtype, tol):
    cfg, w = _model(dtype)
    mr = gu.build_runner(cfg, w, dtype=dtype, device=DEV, max_total_tokens=192, max_running_requests=3)
    # more than 64 rows at once: the prefill-sized GEMM paths, on widths that are multiples of nothing in particular
    long = gu.random_prompts(cfg, [150], seed=4)
    want = {k: ref.forward(gu.public(cfg), w, p) for k, p in long.items()}
    gu.replay_and_compare(mr, cfg, w, long, [[("r0", 150)]], tol, want_all=want)
    gu.replay_and_compare(mr, cfg, w, long, [[("r0", 71)], [("r0", 2)], [("r0", 77)]], tol, want_all=want)
    p = gu.random_prompts(cfg, [23], seed=0)
    want = {k: ref.forward(gu.public(cfg), w, x) for k, x in p.items()}
    gu.replay_and_compare(mr, cfg, w, p, [[("r0", 23)]], tol, want_all=want)
    gu.replay_and_compare(mr, cfg, w, p, [[("r0", 1)] for _ in range(23)], tol, want_all=want)
    gu.replay_and_compare(mr, cfg, w, p, [[("r0", k)] for k in (2, 2, 3, 5, 2, 7, 1, 1)], tol, want_all=want)
    prompts = gu.random_prompts(cfg, [17, 9, 1, 12, 20, 6], seed=7)
    want = {k: ref.forward(gu.public(cfg), w, x) for k, x in prompts.items()}
    sched = [[("r0", 5), ("r1", 2)], [("r0", 1), ("r1", 7), ("r2", 1)], [("r0", 4), ("r3", 3)], [("r3", 1)],
             [("r0", 1), ("r3", 1)], [("r0", 6), ("r3", 7), ("r4", 2)], [("r4", 1), ("r5", 1)], [("r4", 1), ("r5", 1)],
             [("r4", 9), ("r5", 4)], [("r4", 1)], [("r4", 6)]]
    for _ in range(2):        # the second pass runs on used slots, rows, matrices and convolution inputs
        gu.replay_and_compare(mr, cfg, w, prompts, sched, tol, want_all=want)
        assert gu.pools_are_whole(mr)


@pytest.mark.parametrize("dtype,tol", CASES)
@pytest.mark.parametrize("page_size", [1, 16])
def test_long_decode_on_other_sizes(dtype, tol, page_size):
    """Sizes unlike the small default, on the matrix-core paths in bf16: attention heads of 64 and 32 with values of 32 and
    64, 8 query heads on 2 key heads, a window that decoded tokens leave behind, delta-rule heads of 64 x 32 on shared keys,
    16 experts in 4 groups, a 150-token decode over pages of 16, two requests side by side."""
    every = dtype != "float32"
    layers = [(gu.parallel(heads=8, kv_heads=2, dim=32, vdim=64, window=48, scale=0.18, conv=4, r_heads=4, r_kv_heads=2, r_dim=64,
                           r_vdim=32, r_conv=2, decay_rank=8, gate_rank=4),
               gu.moe(experts=16, top=16 if every else 4, count=4, keep=4 if every else 2, ff=64)),
              (gu.lightning(heads=3, dim=32, vdim=64, decay=(0.99, 0.9, 1.0)), gu.dense(96)),
              (gu.parallel(heads=2, kv_heads=2, dim=64, vdim=32, window=100, scale=0.12, conv=3, r_heads=2, r_kv_heads=1, r_dim=32,
                           r_vdim=64, r_conv=4, decay_rank=16, gate_rank=16), None),
              (gu.lightning(heads=2, dim=64, vdim=32, decay=(0.97, 0.8)), gu.moe(experts=8, top=8, count=1, keep=1, ff=32))]
    cfg = gu.make_config(layers=layers, width=128, vocab=97, taps=4, embed_scale=2.0, logit_scale=0.3)
    w = gu.make_weights(cfg, seed=21)
    mr = gu.build_runner(cfg, w, dtype=dtype, device=DEV, max_total_tokens=512, max_running_requests=2, page_size=page_size)
    p = gu.random_prompts(cfg, [190, 75], seed=3)
    want = {k: ref.forward(gu.public(cfg), w, x) for k, x in p.items()}
    sched = [[("r0", 40), ("r1", 2)]] + [[("r0", 1), ("r1", 1)] for _ in range(73)] + [[("r0", 1)] for _ in range(77)]
    gu.replay_and_compare(mr, cfg, w, p, sched, tol, want_all=want)
    gu.replay_and_compare(mr, cfg, w, p, [[("r1", 75)], [("r0", 100)], [("r0", 31)], [("r0", 2)], [("r0", 57)]], tol, want_all=want)
    assert gu.pools_are_whole(mr)


@pytest.mark.parametrize("dtype,tol", CASES)
def test_sizes_that_are_multiples_of_nothing_in_particular(dtype, tol):
    """Five layers in another order, without feed-forward at the end: attention heads of 48 with values of 80 (the
    vector-ALU kernel in bf16 too) and of 128 / 128, 8 query heads on 2 key heads, windows of 7, 33 and 200, convolutions
    of 2 to 5 taps, delta-rule heads of 24 x 40 on shared keys and of 128 x 128, five decays incl. 1, eight experts in four
    groups, a width of 192; a 260-token prompt beside shorter ones, portions beside single tokens, the pools used twice."""
    every = dtype != "float32"
    layers = [(gu.lightning(heads=5, dim=48, vdim=24, decay=(0.5, 0.9, 0.99, 0.999, 1.0)),
               gu.moe(experts=8, top=8 if every else 3, count=4, keep=4 if every else 2, ff=40)),
              (gu.parallel(heads=8, kv_heads=2, dim=48, vdim=80, window=33, scale=0.2, conv=2, r_heads=6, r_kv_heads=3, r_dim=24, r_vdim=40,
                           r_conv=5, decay_rank=12, gate_rank=20), gu.dense(100)),
              (gu.parallel(heads=4, kv_heads=4, dim=128, vdim=128, window=200, scale=0.09, conv=4, r_heads=2, r_kv_heads=1, r_dim=128,
                           r_vdim=128, r_conv=4, decay_rank=24, gate_rank=24), gu.moe(experts=4, top=4 if every else 2, count=2, keep=2, ff=96)),
              (gu.lightning(heads=8, dim=32, vdim=32, decay=[0.9 + 0.01 * i for i in range(8)]), None),
              (gu.parallel(heads=3, kv_heads=1, dim=64, vdim=32, window=7, scale=0.125, conv=3, r_heads=3, r_kv_heads=3, r_dim=64, r_vdim=64,
                           r_conv=3, decay_rank=8, gate_rank=8), None)]
    cfg = gu.make_config(layers=layers, width=192, vocab=1000, taps=2, embed_scale=9.0, logit_scale=0.1, eps=1e-6)
    w = gu.make_weights(cfg, seed=5)
    mr = gu.build_runner(cfg, w, dtype=dtype, device=DEV, max_total_tokens=448, max_running_requests=4)
    p = gu.random_prompts(cfg, [260, 90, 3, 60], seed=8)
    want = {k: ref.forward(gu.public(cfg), w, x) for k, x in p.items()}
    gu.replay_and_compare(mr, cfg, w, {"r0": p["r0"]}, [[("r0", 260)]], tol, want_all=want)
    sched = [[("r0", 64), ("r1", 64), ("r2", 2)], [("r0", 29), ("r1", 2), ("r2", 1), ("r3", 16)], [("r0", 128), ("r1", 3), ("r3", 3)],
             [("r0", 2), ("r1", 16), ("r3", 35)], [("r0", 30), ("r1", 4), ("r3", 5)]] + [[("r0", 1), ("r1", 1), ("r3", 1)]] + [[("r0", 1)]] * 6
    for _ in range(2):
        gu.replay_and_compare(mr, cfg, w, p, sched, tol, want_all=want)
        assert gu.pools_are_whole(mr)


@pytest.mark.parametrize("dtype,tol", CASES)
def test_equal_and_unit_sizes(dtype, tol):
    """The sizes of the CPU test of this name, with heads of 8 where it has heads of 4: a head of 4 values divided by its
    root mean square turns bf16 noise into a large change of direction whenever the head's output is near zero."""
    layers = [(gu.parallel(heads=2, kv_heads=2, dim=8, vdim=8, window=1, conv=2, r_heads=1, r_kv_heads=1, r_dim=8, r_vdim=8, r_conv=2,
                           decay_rank=1, gate_rank=1), gu.moe(experts=3, top=3 if dtype != "float32" else 1, count=1, keep=1, ff=8)),
              (gu.lightning(heads=1, dim=8, vdim=8, decay=(1.0,)), None),
              (gu.parallel(heads=3, kv_heads=1, dim=8, vdim=8, window=3, conv=2, r_heads=3, r_kv_heads=3, r_dim=8, r_vdim=8, r_conv=2),
               gu.moe(experts=4, top=4, count=4, keep=4, ff=4)),
              (gu.lightning(heads=2, dim=8, vdim=8, decay=(0.5, 0.5)), gu.dense(16))]
    cfg = gu.make_config(layers=layers, width=16, vocab=16, taps=2, embed_scale=1.0, logit_scale=1.0)
    w = gu.make_weights(cfg, seed=11)
    prompts = gu.random_prompts(cfg, [14, 5], seed=1)
    mr = gu.build_runner(cfg, w, dtype=dtype, device=DEV, max_total_tokens=32)
    gu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 3), ("r1", 1)], [("r0", 1), ("r1", 1)], [("r0", 10), ("r1", 3)]], tol)
    assert gu.pools_are_whole(mr)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_scheduler(dtype):
    """The engine's own entry point, prompts chunked and decode tokens riding prefill batches.  fp32 must give the
    oracle's tokens; bf16 must give the same tokens whether a prompt is chunked or not, up to a near-tie."""
    from sglang_custom_amd.managers.schedule_batch import Req
    from sglang_custom_amd.managers.scheduler import Scheduler
    from sglang_custom_amd.sampling.sampling_params import SamplingParams

    cfg, w = _model(dtype)
    prompts = gu.random_prompts(cfg, [11, 3, 7, 15, 1], seed=9)
    outs = []
    for chunk, mixed in ((None, False), (6, True)):
        mr = gu.build_runner(cfg, w, dtype=dtype, device=DEV, max_total_tokens=96, max_running_requests=3,
                             chunked_prefill_size=chunk, enable_mixed_chunk=mixed)
        sch = Scheduler(mr)
        for k, p in prompts.items():
            sch.add_request(Req(k, p, SamplingParams(temperature=0, max_new_tokens=6)))
        done = sch.run_until_done()
        outs.append({k: done[k].output_ids for k in prompts})
        assert gu.pools_are_whole(mr)
    if dtype == "float32":
        for k, p in prompts.items():
            assert outs[0][k] == outs[1][k] == ref.greedy(gu.public(cfg), w, p, 6), k
    else:
        same = sum(outs[0][k] == outs[1][k] for k in prompts)
        assert same >= len(prompts) - 1


@pytest.mark.parametrize("dtype,tol", CASES)
def test_command_line_replay_of_a_model_folder(tmp_path, dtype, tol):
    """bin/trace_run as a user starts it: a model folder on disk, steps on standard input, logits in files; four live
    requests at most, a pool that the requests' total would not fit into."""
    import json
    import os
    import subprocess
    import sys

    import numpy as np

    from test_seturax_gpu import _write_model_folder

    every = dtype != "float32"
    layers = [(gu.lightning(heads=2, dim=16, vdim=32, decay=(0.95, 0.999)), gu.moe(experts=4, top=4 if every else 2, count=2, keep=2 if every else 1, ff=48)),
              (gu.parallel(heads=6, kv_heads=3, dim=32, vdim=32, window=24, conv=3, r_heads=4, r_kv_heads=4, r_dim=16, r_vdim=16, r_conv=4,
                           decay_rank=7, gate_rank=7), gu.dense(80)),
              (gu.parallel(heads=2, kv_heads=1, dim=16, vdim=48, window=50, conv=4, r_heads=2, r_kv_heads=1, r_dim=32, r_vdim=32, r_conv=3),
               gu.moe(experts=6, top=6 if every else 3, count=3, keep=3 if every else 2, ff=24))]
    cfg = gu.make_config(layers=layers, width=64, vocab=83, taps=4, embed_scale=5.0, logit_scale=0.25)
    w = gu.make_weights(cfg, seed=17)
    _write_model_folder(tmp_path, gu.public(cfg), w)
    prompts = gu.random_prompts(cfg, [70, 33, 1, 64, 40], seed=6)
    sched = [[("r0", 40), ("r1", 2)], [("r0", 1), ("r1", 30), ("r2", 1), ("r3", 7)], [("r0", 29), ("r1", 1), ("r3", 57)],
             [("r4", 2)], [("r4", 1)], [("r4", 37)]]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    lines, want, at = [], [], {k: 0 for k in prompts}
    full = {k: ref.forward(gu.public(cfg), w, p) for k, p in prompts.items()}
    for n, step in enumerate(sched):
        entries, rows, end = [], [], []
        for name, cnt in step:
            lo, hi = at[name], at[name] + cnt
            asked = list(range(0, cnt, 3)) + ([cnt - 1] if (cnt - 1) % 3 else [])
            entries.append({"id": name, "tokens": prompts[name][lo:hi], "want": asked})
            rows.append(full[name][lo:hi][asked])
            at[name] = hi
            if hi == len(prompts[name]):
                end.append(name)
        lines.append(json.dumps({"step": n, "entries": entries, "end": end}))
        want.append(torch.cat(rows))
    lines.append(json.dumps({"step": len(sched), "entries": [], "end": []}))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(tmp_path), "--dtype", dtype, "--out", str(out),
                        "--max-tokens", "192"], input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=300, cwd=root)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [x for x in r.stdout.split("\n") if x.startswith("done")] == [f"done {n}" for n in range(len(sched) + 1)]
    errors = []
    for n, expect in enumerate(want):
        got = torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, cfg["vocab"]).copy())
        assert got.shape == expect.shape
        errors.append(gu.row_errors(got, expect))
    assert gu.within(torch.cat(errors), tol, dtype != "float32"), [float(e.max()) for e in errors]
    assert not (out / f"{len(sched)}.f32").exists()
