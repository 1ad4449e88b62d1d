"""Fudonex on the GPU: every HIP kernel the family added or extended against the plain functions of oracle/fudonex_ref.py
(fudonex_cases.py holds the cases), then the whole engine (ModelRunner, pools, TraceReplayer, Scheduler) in fp32 and bf16
against the whole-sequence oracle.  Where random numbers would hide a fault -- a key at the window's edge, a block that is
just seen and one that is not yet, tokens between the window and their block, a far block among dozens, a value written
hundreds of tokens back, the first tokens of a sequence, stale averages and stale state in reused slots -- the inputs are
built so that it shows."""
import pytest
import torch

import fudonex_cases as cases
import fudonex_util as fu
from oracle import fudonex_ref as ref

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
def test_output_norm_with_layer_scale(dtype, D):
    cases.check_output_norm_add(ops(), DEV, dtype, D=D)
    cases.check_output_norm_add(ops(), DEV, dtype, D=D, mult=1.0, T=1)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gate_then_group_norm(dtype):
    cases.check_gated_group_norm(ops(), DEV, dtype)
    cases.check_gated_group_norm(ops(), DEV, dtype, T=3, D=256, parts_list=(1, 4, 256))


@pytest.mark.parametrize("dtype", DTYPES)
def test_scaled_rotation(dtype):
    cases.check_scaled_frequencies()
    cases.check_scaled_rotation(ops(), DEV, dtype)
    cases.check_scaled_rotation(ops(), DEV, dtype, H=1, d=64, rot_dims=64)
    cases.check_scaled_rotation(ops(), DEV, dtype, H=5, d=48, rot_dims=2)
    cases.check_qkv_norms_one_launch(ops(), DEV, dtype)
    cases.check_qkv_norms_one_launch(ops(), DEV, dtype, H=8, G=1, d=128, dv=64, rot_dims=128)
    cases.check_qkv_norms_one_launch(ops(), DEV, dtype, H=1, G=1, d=6, dv=200, rot_dims=0, T=3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_convolution_with_bias(dtype):
    cases.check_conv_bias(ops(), DEV, dtype)
    cases.check_conv_bias(ops(), DEV, dtype, C=256)
    cases.check_conv_bias(ops(), DEV, dtype, C=12, T=14)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,N,dv", [(4, 2, 10, 20), (6, 2, 32, 40), (2, 2, 64, 64), (3, 3, 1, 1), (8, 2, 128, 32), (1, 1, 200, 40)])
def test_state_space_recurrence(dtype, H, G, N, dv):
    for cuts, tail in (((45,), 0), ((20, 2, 1, 22), 0), ((3, 40, 1, 1), 2), ((1,) * 45, 45), ((17, 16, 12), 0)):
        cases.check_state_space(ops(), DEV, dtype, H=H, G=G, N=N, dv=dv, cuts=cuts, decode_tail=tail)
    cases.check_state_space(ops(), DEV, dtype, H=H, G=G, N=N, dv=dv, cuts=(44, 1), decode_tail=1, with_skip=False)


@pytest.mark.parametrize("dtype", DTYPES)
def test_state_space_far_write_and_stale_slot(dtype):
    cases.check_state_space_planted(ops(), DEV, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,dk,dv", [(4, 2, 12, 20), (4, 2, 64, 48), (2, 2, 128, 128), (6, 1, 1, 3), (3, 3, 40, 70)])
def test_delta_rule_with_a_decay_per_head(dtype, H, G, dk, dv):
    for cuts, tail in (((45,), 0), ((20, 2, 1, 22), 0), ((3, 40, 1, 1), 2), ((1,) * 45, 45)):
        cases.check_delta_rule(ops(), DEV, dtype, H=H, G=G, dk=dk, dv=dv, cuts=cuts, decode_tail=tail)


@pytest.mark.parametrize("dtype", DTYPES)
def test_delta_rule_far_write_replaced_and_forgotten(dtype):
    cases.check_delta_rule_planted(ops(), DEV, dtype)


# head shapes: matrix-core tiles (widths that are multiples of 32 / 16), the vector-ALU kernel (48 / 24, 20 / 12), many heads on one key head
SHAPES = [(4, 2, 32, 32), (6, 3, 48, 24), (8, 2, 128, 128), (16, 1, 64, 32), (2, 2, 20, 12), (3, 1, 96, 64), (40, 1, 32, 16)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,d,dv", SHAPES)
def test_attention_over_window_and_blocks(dtype, H, G, d, dv):
    o = ops()
    for window, pool, T, cuts, page, tail, splits in ((40, 8, 150, (150,), 1, 0, 1), (40, 8, 150, (17, 2, 100, 30, 1), 1, 1, 1),
                                                     (88, 8, 300, (290,) + (1,) * 10, 16, 10, 3), (7, 3, 100, (50, 2, 47, 1), 6, 1, 2),
                                                     (33, 5, 130, (64, 64, 2), 4, 0, 1), (1, 1, 70, (35, 34, 1), 1, 1, 2),
                                                     (16, 64, 200, (200,), 64, 0, 1), (200, 4, 90, (88, 1, 1), 1, 2, 2)):
        cases.check_pooled_attention(o, DEV, dtype, H=H, G=G, d=d, dv=dv, T=T, window=window, pool=pool, cuts=cuts, page=page,
                                     decode_tail=tail, splits=splits)
    cases.check_pooled_attention(o, DEV, dtype, H=H, G=G, d=d, dv=dv, T=90, window=30, pool=0, cuts=(60, 30), with_gate=False)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("d", [32, 48])
def test_attention_block_edges_gaps_and_far_blocks(dtype, d):
    for W, P, page in ((24, 8, 1), (24, 8, 64), (56, 16, 1), (6, 4, 8), (40, 32, 1), (33, 3, 4)):
        cases.check_pooled_attention_planted(ops(), DEV, dtype, d=d, W=W, P=P, page=page)


# ---------------------------------------------------------------------------------------------- the engine
CASES = [("float32", 3e-5), ("bfloat16", 6e-2)]


def _model(dtype, **kw):
    """fp32: the CPU tests' small model.  bf16: the same order of layers with twice the widths.  Both recurrent mixers norm
    their own output before the layer norms it again, so a read-out whose terms nearly cancel is divided by its own small
    size twice; over 24 values that turns 16-bit rounding of the inputs into a visible change of one row in a few dozen (the
    CPU stand-ins in bf16 show the same rows), over 64 and more it stays inside the tolerance."""
    if dtype == "float32":
        cfg = fu.make_config(**kw)
        return cfg, fu.make_weights(cfg, seed=3)
    layers = [(fu.attention(heads=4, kv_heads=2, dim=32, vdim=16, window=7, pool=3), fu.dense(96)),
              (fu.mamba2(heads=4, vdim=16, state=16, groups=2, norm_groups=2, conv=3), fu.dense(64)),
              (fu.delta(heads=4, kv_heads=2, dim=16, vdim=16, conv=4), None),
              (fu.attention(heads=6, kv_heads=2, dim=32, vdim=16, window=5, pool=2, scale=0.5, rot_dims=16, scaling=False, kv_from=0), fu.dense(64)),
              (fu.attention(heads=2, kv_heads=1, dim=24, vdim=40, window=9, pool=2, rot_dims=4, base=50.0), fu.dense(48)),
              (fu.mamba2(heads=3, vdim=24, state=8, groups=1, norm_groups=1, conv=2), None)]
    cfg = fu.make_config(layers=layers, width=96, vocab=101, **kw)
    return cfg, fu.make_weights(cfg, seed=3)


@pytest.mark.parametrize("dtype,tol", CASES)
@pytest.mark.parametrize("kind", ["attention", "mamba2", "delta"])
def test_each_mixer_alone(dtype, tol, kind):
    mixer = dict(attention=fu.attention(window=20, pool=8), mamba2=fu.mamba2(), delta=fu.delta())[kind]
    cfg = fu.make_config(layers=[(mixer, None)])
    w = fu.make_weights(cfg, seed=1)
    prompts = fu.random_prompts(cfg, [90])
    mr = fu.build_runner(cfg, w, dtype=dtype, device=DEV)
    fu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 90)]], tol)
    fu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 37)], [("r0", 2)], [("r0", 40)]] + [[("r0", 1)] for _ in range(11)], tol)
    assert fu.pools_are_whole(mr)


@pytest.mark.parametrize("dtype,tol", CASES)
def test_portions_and_batches(dtype, tol):
    cfg, w = _model(dtype)
    prompts = fu.random_prompts(cfg, [27, 9, 1, 12, 30, 6], seed=7)
    sched = [[("r0", 5), ("r1", 2)], [("r0", 1), ("r1", 7), ("r2", 1)], [("r0", 4), ("r3", 3)], [("r3", 1)],
             [("r0", 1), ("r3", 1)], [("r0", 16), ("r3", 7), ("r4", 2)], [("r4", 1), ("r5", 1)], [("r4", 1), ("r5", 1)],
             [("r4", 19), ("r5", 4)], [("r4", 1)], [("r4", 6)]]
    want = {k: ref.forward(cfg, w, p) for k, p in prompts.items()}
    for page in (1, 6):
        mr = fu.build_runner(cfg, w, dtype=dtype, device=DEV, max_total_tokens=72, max_running_requests=3, page_size=page)
        for _ in range(2):       # the second time over used slots, averages and state
            fu.replay_and_compare(mr, cfg, w, prompts, sched, tol, want_all=want)
            assert fu.pools_are_whole(mr)


@pytest.mark.parametrize("dtype,tol", CASES)
def test_long_decode_past_windows_and_blocks(dtype, tol):
    """Other sizes than the small default's: heads of 64 and 32 on the matrix cores in bf16, a window of 48 with blocks of 16,
    a layer that reads the same cache under a window of 20 with blocks of 8, and a window of 20 with blocks of 5, all of which
    a 170-token decode passes several times; pages of 16."""
    layers = [(fu.attention(heads=4, kv_heads=2, dim=64, vdim=32, window=48, pool=16, scale=0.125, rot_dims=32, base=10000.0,
                            scaling=dict(factor=8.0, original=64, fast=8.0, slow=1.0)), fu.dense(96)),
              (fu.mamba2(heads=4, vdim=32, state=16, groups=2, norm_groups=2, conv=4), fu.dense(64)),
              (fu.attention(heads=4, kv_heads=2, dim=64, vdim=32, window=20, pool=8, scale=0.2, rot_dims=32, base=10000.0,
                            scaling=dict(factor=8.0, original=64, fast=8.0, slow=1.0), kv_from=0), None),
              (fu.delta(heads=4, kv_heads=2, dim=32, vdim=32, conv=3), fu.dense(64)),
              (fu.attention(heads=3, kv_heads=1, dim=32, vdim=48, window=20, pool=5, scale=0.18, rot_dims=16), fu.dense(64))]
    cfg = fu.make_config(layers=layers, width=128, vocab=211, embed_scale=6.0, residual_mult=0.7, softcap=20.0, eps=1e-6)
    w = fu.make_weights(cfg, seed=5)
    mr = fu.build_runner(cfg, w, dtype=dtype, device=DEV, max_total_tokens=512, max_running_requests=4, page_size=16)
    p = fu.random_prompts(cfg, [260, 90, 3, 60], seed=8)
    want = {k: ref.forward(cfg, w, x) for k, x in p.items()}
    fu.replay_and_compare(mr, cfg, w, {"r0": p["r0"]}, [[("r0", 260)]], tol, want_all=want)
    fu.replay_and_compare(mr, cfg, w, {"r0": p["r0"]}, [[("r0", 90)]] + [[("r0", 1)]] * 170, tol, want_all=want)
    sched = [[("r0", 64), ("r1", 64), ("r2", 2)], [("r0", 29), ("r1", 2), ("r2", 1), ("r3", 16)], [("r0", 128), ("r1", 3), ("r3", 3)],
             [("r0", 2), ("r1", 16), ("r3", 35)], [("r0", 30), ("r1", 4), ("r3", 5)]] + [[("r0", 1), ("r1", 1), ("r3", 1)]] + [[("r0", 1)]] * 6
    for _ in range(2):
        fu.replay_and_compare(mr, cfg, w, p, sched, tol, want_all=want)
        assert fu.pools_are_whole(mr)


@pytest.mark.parametrize("dtype,tol", CASES)
def test_sizes_that_are_multiples_of_nothing(dtype, tol):
    """Width 100, vocabulary 77, heads of 20 / 12 / 36, a state of 7, 3 and 5 taps, blocks of 7 and 5 under windows of 11 and
    9, pages of 5: no 16-byte row anywhere in 16 bits, no whole tile, no whole block per page."""
    layers = [(fu.attention(heads=3, kv_heads=1, dim=20, vdim=12, window=11, pool=7, scale=0.22, rot_dims=10, base=77.0), fu.dense(50)),
              (fu.mamba2(heads=3, vdim=12, state=7, groups=1, norm_groups=3, conv=3), fu.dense(30)),
              (fu.delta(heads=3, kv_heads=1, dim=20, vdim=36, conv=5), fu.dense(70)),
              (fu.attention(heads=6, kv_heads=1, dim=20, vdim=12, window=9, pool=5, scale=0.3, rot_dims=10, base=77.0, kv_from=0), None)]
    cfg = fu.make_config(layers=layers, width=100, vocab=77, embed_scale=2.5, residual_mult=0.8, softcap=9.0)
    w = fu.make_weights(cfg, seed=21)
    mr = fu.build_runner(cfg, w, dtype=dtype, device=DEV, max_total_tokens=200, max_running_requests=3, page_size=5)
    p = fu.random_prompts(cfg, [83, 41, 6], seed=4)
    want = {k: ref.forward(cfg, w, x) for k, x in p.items()}
    sched = [[("r0", 33), ("r1", 2)], [("r0", 2), ("r1", 30), ("r2", 1)], [("r0", 40), ("r1", 1), ("r2", 5)], [("r0", 1), ("r1", 1)],
             [("r0", 1), ("r1", 7)]] + [[("r0", 1)]] * 6
    for _ in range(2):
        fu.replay_and_compare(mr, cfg, w, p, sched, tol, want_all=want)
        assert fu.pools_are_whole(mr)


@pytest.mark.parametrize("dtype,tol", CASES)
def test_equal_and_unit_sizes(dtype, tol):
    """The sizes of the CPU test of this name, with heads of 8 where it has heads of 4: a head of 4 values divided by its
    root mean square turns bf16 noise into a large change of direction whenever the head's output is near zero.  At width 16
    every sublayer's output is divided by the root mean square of sixteen numbers, seven layers in a row: the 16-bit run is
    held to twice the usual distance here."""
    if dtype != "float32":
        tol = 2 * tol
    layers = [(fu.attention(heads=2, kv_heads=2, dim=8, vdim=8, window=1, pool=1, rot_dims=8, scaling=False), fu.dense(8)),
              (fu.mamba2(heads=1, vdim=8, state=4, groups=1, norm_groups=1, conv=2), None),
              (fu.delta(heads=1, kv_heads=1, dim=8, vdim=8, conv=2), None),
              (fu.attention(heads=3, kv_heads=1, dim=8, vdim=8, window=3, pool=3, rot_dims=0), fu.dense(16)),
              (fu.mamba2(heads=2, vdim=8, state=8, groups=2, norm_groups=2, conv=2), fu.dense(16)),
              (fu.attention(heads=2, kv_heads=2, dim=8, vdim=8, window=1, pool=1, rot_dims=8, scaling=False, kv_from=0), None),
              (fu.delta(heads=3, kv_heads=3, dim=8, vdim=8, conv=4), fu.dense(4))]
    cfg = fu.make_config(layers=layers, width=16, vocab=16, embed_scale=1.0, residual_mult=1.0, softcap=None)
    w = fu.make_weights(cfg, seed=11)
    prompts = fu.random_prompts(cfg, [14, 5], seed=1)
    mr = fu.build_runner(cfg, w, dtype=dtype, device=DEV, max_total_tokens=32)
    fu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 3), ("r1", 1)], [("r0", 1), ("r1", 1)], [("r0", 10), ("r1", 3)]], tol)
    assert fu.pools_are_whole(mr)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_scheduler(dtype):
    """The engine's own entry point, prompts chunked and decode tokens riding prefill batches.  fp32 must give the
    oracle's tokens; bf16 must give the same tokens whether a prompt is chunked or not, up to a near-tie."""
    from sglang_custom_amd.managers.schedule_batch import Req
    from sglang_custom_amd.managers.scheduler import Scheduler
    from sglang_custom_amd.sampling.sampling_params import SamplingParams

    cfg, w = _model(dtype)
    prompts = fu.random_prompts(cfg, [11, 3, 7, 15, 1], seed=9)
    outs = []
    for chunk, mixed in ((None, False), (6, True)):
        mr = fu.build_runner(cfg, w, dtype=dtype, device=DEV, max_total_tokens=96, max_running_requests=3,
                             chunked_prefill_size=chunk, enable_mixed_chunk=mixed)
        sch = Scheduler(mr)
        for k, p in prompts.items():
            sch.add_request(Req(k, p, SamplingParams(temperature=0, max_new_tokens=6)))
        done = sch.run_until_done()
        outs.append({k: done[k].output_ids for k in prompts})
        assert fu.pools_are_whole(mr)
    if dtype == "float32":
        for k, p in prompts.items():
            assert outs[0][k] == outs[1][k] == ref.greedy(cfg, w, p, 6), k
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

    layers = [(fu.mamba2(heads=2, vdim=32, state=16, groups=1, norm_groups=4, conv=4), fu.dense(48)),
              (fu.attention(heads=6, kv_heads=3, dim=32, vdim=32, window=24, pool=8, scale=0.2, rot_dims=16), fu.dense(80)),
              (fu.delta(heads=2, kv_heads=1, dim=32, vdim=32, conv=3), None),
              (fu.attention(heads=3, kv_heads=3, dim=32, vdim=32, window=10, pool=8, scale=0.3, rot_dims=16, kv_from=1), fu.dense(24))]
    cfg = fu.make_config(layers=layers, width=64, vocab=83, embed_scale=5.0, residual_mult=0.25, softcap=8.0)
    w = fu.make_weights(cfg, seed=17)
    _write_model_folder(tmp_path, cfg, w)
    prompts = fu.random_prompts(cfg, [70, 33, 1, 64, 40], seed=6)
    sched = [[("r0", 40), ("r1", 2)], [("r0", 1), ("r1", 30), ("r2", 1), ("r3", 7)], [("r0", 29), ("r1", 1), ("r3", 57)],
             [("r4", 2)], [("r4", 1)], [("r4", 37)]]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    lines, want, at = [], [], {k: 0 for k in prompts}
    full = {k: ref.forward(cfg, w, p) for k, p in prompts.items()}
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
        errors.append(fu.row_errors(got, expect))
    assert fu.within(torch.cat(errors), tol, dtype != "float32"), [float(e.max()) for e in errors]
    assert not (out / f"{len(sched)}.f32").exists()
