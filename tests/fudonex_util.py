"""Shared pieces of the Fudonex tests: small random models in checkpoint form and the replay of a schedule with every
logit compared against the whole-sequence oracle (oracle/fudonex_ref.py)."""
import torch

from gatarax_util import row_errors, within
from oracle import fudonex_ref as ref
from seturax_util import build_runner, random_prompts, rel_err  # noqa: F401  (generic helpers)


def pools_are_whole(runner) -> bool:
    """Every KV slot, request row and state slot (where the model has state) is back."""
    mr = runner
    st = mr.req_to_token_pool.state_pool
    return (mr.token_to_kv_pool_allocator.available_size() == mr.max_total_num_tokens
            and mr.req_to_token_pool.available_size() == mr.req_to_token_pool.size
            and (st is None or st.available_size() == st.size))


def attention(heads=4, kv_heads=2, dim=16, vdim=8, window=7, pool=3, scale=0.3, rot_dims=8, base=500.0, scaling=True, kv_from=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, mask=dict(size=window, pool=pool))
    if rot_dims:
        m["rot"] = dict(base=base, dims=rot_dims)
        if scaling:
            m["rot"]["scaling"] = dict(factor=4.0, original=16, fast=2.0, slow=0.5) if scaling is True else dict(scaling)
    if kv_from is not None:
        m["kv_from"] = kv_from
    return dict(type="attention", mixer=m)


def mamba2(heads=4, vdim=6, state=10, groups=2, norm_groups=3, conv=3):
    return dict(type="mamba2", mixer=dict(heads=heads, vdim=vdim, state=state, groups=groups, norm_groups=norm_groups, conv=conv))


def delta(heads=4, kv_heads=2, dim=12, vdim=10, conv=4):
    return dict(type="delta", mixer=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv))


def dense(ff=40):
    return dict(kind="dense", ff=ff)


def default_layers():
    """Every mixer, an attention layer that borrows another's keys under a window and a block length of its own, a layer without
    feed-forward; unlike sizes throughout."""
    return [(attention(), dense()), (mamba2(), dense(24)), (delta(), None),
            (attention(heads=6, kv_heads=2, dim=16, vdim=8, window=5, pool=2, scale=0.5, rot_dims=16, scaling=False, kv_from=0), dense(32)),
            (attention(heads=2, kv_heads=1, dim=12, vdim=20, window=9, pool=2, rot_dims=4, base=50.0), dense(16)),
            (mamba2(heads=3, vdim=8, state=5, groups=1, norm_groups=1, conv=2), None)]


def make_config(layers=None, width=48, vocab=53, embed_scale=2.0, residual_mult=0.6, softcap=12.0, eps=1e-5):
    """layers: list of (mixer spec, mlp spec or None)."""
    if layers is None:
        layers = default_layers()
    cfg = dict(architecture="Fudonex", vocab=vocab, width=width, norm=dict(eps=eps), embedding=dict(scale=embed_scale),
               residual_mult=residual_mult,
               layers=[dict(type=m["type"], mixer={k: (dict(v) if isinstance(v, dict) else v) for k, v in m["mixer"].items()}, mlp=f)
                       for m, f in layers])
    if softcap:
        cfg["logit_softcap"] = softcap
    return cfg


def make_weights(cfg, seed=0):
    """Checkpoint-named tensors with bf16-representable values, so that a bf16 and an fp32 run read the same numbers."""
    g = torch.Generator().manual_seed(seed)
    D, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, std=1.0, mean=0.0):
        return (mean + std * torch.randn(*shape, generator=g)).to(torch.bfloat16)

    w = {"embed": rnd(V, D, std=1.0 / cfg["embedding"]["scale"]), "final.norm": rnd(D, std=0.1)}
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}.", spec["mixer"]
        x = p + "mix."
        w[p + "norm1"] = rnd(D, std=0.1)
        w[p + "ls1"] = rnd(D, std=0.2, mean=1.0)
        if spec["type"] == "attention":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            names = [("q", H * d)] + ([("k", G * d), ("v", G * dv)] if m.get("kv_from") is None else [])
            for n, rows in names:
                w[x + n] = rnd(rows, D, std=D ** -0.5)
                w[x + n + ".b"] = rnd(rows, std=0.3)
            w[x + "q.norm"] = rnd(d, std=0.1, mean=1.0)
            if m.get("kv_from") is None:
                w[x + "k.norm"] = rnd(d, std=0.1, mean=1.0)
            w[x + "sink"] = rnd(H, std=1.0)
            w[x + "g"] = rnd(H, D, std=2 * D ** -0.5)
            w[x + "o"] = rnd(D, H * dv, std=(H * dv) ** -0.5)
        elif spec["type"] == "mamba2":
            H, dv, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            inner, ch = H * dv, H * dv + 2 * G * N
            w[x + "in"] = rnd(inner + ch + H, D, std=D ** -0.5)
            w[x + "conv"] = rnd(ch, m["conv"], std=0.6)
            w[x + "conv.b"] = rnd(ch, std=0.2)
            w[x + "dt_bias"] = rnd(H, std=0.5, mean=-1.0)
            w[x + "A_log"] = rnd(H, std=0.5)
            w[x + "D"] = rnd(H, std=0.3, mean=1.0)
            w[x + "norm"] = rnd(inner, std=0.1, mean=1.0)
            w[x + "o"] = rnd(D, inner, std=inner ** -0.5)
        else:
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            for n, rows in (("q", G * d), ("k", G * d), ("v", H * dv)):
                w[x + n] = rnd(rows, D, std=D ** -0.5)
                w[x + n + ".conv"] = rnd(rows, m["conv"], std=0.6)
            w[x + "b"] = rnd(H, D, std=D ** -0.5)
            w[x + "a"] = rnd(H, D, std=D ** -0.5)
            w[x + "dt_bias"] = rnd(H, std=0.5, mean=-1.0)
            w[x + "A_log"] = rnd(H, std=0.5)
            w[x + "g"] = rnd(H * dv, D, std=D ** -0.5)
            w[x + "norm"] = rnd(dv, std=0.1, mean=1.0)
            w[x + "o"] = rnd(D, H * dv, std=(H * dv) ** -0.5)
        mlp = spec["mlp"]
        if mlp is not None:
            w[p + "norm2"] = rnd(D, std=0.1)
            w[p + "ls2"] = rnd(D, std=0.2, mean=1.0)
            w[p + "mlp.gate"] = rnd(mlp["ff"], D, std=D ** -0.5)
            w[p + "mlp.up"] = rnd(mlp["ff"], D, std=D ** -0.5)
            w[p + "mlp.down"] = rnd(D, mlp["ff"], std=mlp["ff"] ** -0.5)
    return w


def replay_and_compare(runner, cfg, weights, prompts, schedule, tol, want_all=None):
    """schedule: list of steps, each a list of (request name, token count).  Every token's logits are asked for and
    compared with the oracle's logits of the whole prompt; a request ends with its last token.  Returns the worst error."""
    from sglang_custom_amd.managers.trace_replay import TraceReplayer

    sixteen = runner.dtype != torch.float32
    errors = []
    rp = TraceReplayer(runner)
    want = want_all if want_all is not None else {k: ref.forward(cfg, weights, p) for k, p in prompts.items()}
    at = {k: 0 for k in prompts}
    worst = 0.0
    for step in schedule:
        entries, rows, end = [], [], []
        for name, n in step:
            lo, hi = at[name], at[name] + n
            entries.append(dict(id=name, tokens=prompts[name][lo:hi], want=list(range(n))))
            rows.append(want[name][lo:hi])
            at[name] = hi
            if hi == len(prompts[name]):
                end.append(name)
        got = rp.step(entries, end)
        e = row_errors(got, torch.cat(rows))
        assert float(e.max()) < (3 * tol if sixteen else tol), f"step {step}: logits differ from the whole-sequence oracle by {float(e.max()):.3g} (limit {tol})"
        errors.append(e)
        worst = max(worst, float(e.max()))
    assert all(at[k] == len(p) for k, p in prompts.items()), "the schedule does not cover the prompts"
    assert not rp.live
    assert within(torch.cat(errors), tol, sixteen), f"{int((torch.cat(errors) >= tol).sum())} of {torch.cat(errors).numel()} rows differ by more than {tol}"
    return worst
