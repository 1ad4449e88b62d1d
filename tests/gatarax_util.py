"""Shared pieces of the Gatarax tests: small random models in checkpoint form and the replay of a schedule with every
logit compared against the whole-sequence oracle (oracle/gatarax_ref.py)."""
import torch

from oracle import gatarax_ref as ref
from seturax_util import build_runner, pools_are_whole, random_prompts, rel_err  # noqa: F401  (generic helpers)


def parallel(heads=4, kv_heads=2, dim=16, vdim=8, window=5, scale=0.3, conv=3, r_heads=4, r_kv_heads=2, r_dim=8, r_vdim=12,
             r_conv=4, decay_rank=5, gate_rank=3):
    return dict(type="parallel",
                mixer=dict(left=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv, scale=scale, mask=dict(size=window)),
                           right=dict(heads=r_heads, kv_heads=r_kv_heads, dim=r_dim, vdim=r_vdim, conv=r_conv)),
                _ranks=(decay_rank, gate_rank))


def lightning(heads=3, dim=8, vdim=12, decay=(0.5, 0.9, 0.99)):
    return dict(type="lightning", mixer=dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay)))


def dense(ff=40):
    return dict(kind="dense", ff=ff)


def moe(experts=6, top=2, count=3, keep=2, ff=20):
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top, groups=dict(count=count, keep=keep)))


def default_layers(every_expert=False):
    """Both mixers and both feed-forwards with unlike sizes.  every_expert: each token uses all experts of its mixtures, so
    that a 16-bit run and a float64 oracle cannot part ways over a close call between two scores (the weights still
    differ from token to token)."""
    a, b = (moe(experts=6, top=6, count=3, keep=3), moe(experts=4, top=4, count=1, keep=1)) if every_expert else \
           (moe(), moe(experts=4, top=3, count=1, keep=1))
    return [(parallel(), dense()), (lightning(), a),
            (parallel(heads=2, kv_heads=1, dim=8, vdim=16, window=9, conv=2, r_heads=2, r_kv_heads=2, r_dim=12, r_vdim=4, r_conv=3,
                      decay_rank=2, gate_rank=6), b),
            (lightning(heads=1, dim=20, vdim=4, decay=(0.8,)), None)]


def make_config(layers=None, width=48, vocab=53, taps=3, embed_scale=3.0, logit_scale=0.5, eps=1e-5):
    """layers: list of (mixer spec, mlp spec or None)."""
    if layers is None:
        layers = default_layers()
    cfg = dict(architecture="Gatarax", vocab=vocab, width=width, logit_scale=logit_scale, norm=dict(eps=eps),
               embedding=dict(scale=embed_scale), canon=dict(taps=taps),
               layers=[dict(type=m["type"], mixer={k: (dict(v) if isinstance(v, dict) else v) for k, v in m["mixer"].items()}, mlp=f)
                       for m, f in layers])
    cfg["_ranks"] = [m.get("_ranks") for m, _ in layers]      # read by make_weights only
    return cfg


def public(cfg):
    return {k: v for k, v in cfg.items() if not k.startswith("_")}


def make_weights(cfg, seed=0):
    """Checkpoint-named tensors with bf16-representable values, so that a bf16 and an fp32 run read the same numbers."""
    g = torch.Generator().manual_seed(seed)
    D, V = cfg["width"], cfg["vocab"]
    taps = cfg["canon"]["taps"]

    def rnd(*shape, std=1.0, mean=0.0):
        return (mean + std * torch.randn(*shape, generator=g)).to(torch.bfloat16)

    w = {"embed": rnd(V, D, std=1.0 / cfg["embedding"]["scale"]), "final.norm": rnd(D, std=0.1)}
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}.", spec["mixer"]
        w[p + "norm1"] = rnd(D, std=0.1)
        w[p + "canon1"] = rnd(D, taps, std=0.4)
        if spec["mlp"] is not None:
            w[p + "canon2"] = rnd(D, taps, std=0.4)
        if spec["type"] == "parallel":
            lf, rt = m["left"], m["right"]
            H, G, d, dv = lf["heads"], lf["kv_heads"], lf["dim"], lf["vdim"]
            for n, rows in (("q", H * d), ("k", G * d), ("v", G * dv)):
                w[p + "mix.left." + n] = rnd(rows, D, std=D ** -0.5)
                w[p + "mix.left." + n + ".b"] = rnd(rows, std=0.3)
                w[p + "mix.left." + n + ".conv"] = rnd(rows, lf["conv"], std=0.6)
            w[p + "mix.left.o"] = rnd(D, H * dv, std=(H * dv) ** -0.5)
            w[p + "mix.left.o.b"] = rnd(D, std=0.3)
            H, G, d, dv = rt["heads"], rt["kv_heads"], rt["dim"], rt["vdim"]
            ra, rg = cfg["_ranks"][i]
            for n, rows in (("q", G * d), ("k", G * d), ("v", H * dv)):
                w[p + "mix.right." + n] = rnd(rows, D, std=D ** -0.5)
                w[p + "mix.right." + n + ".conv"] = rnd(rows, rt["conv"], std=0.6)
            w[p + "mix.right.b"] = rnd(H, D, std=D ** -0.5)
            w[p + "mix.right.a1"] = rnd(ra, D, std=D ** -0.5)
            w[p + "mix.right.a2"] = rnd(H * d, ra, std=ra ** -0.5)
            w[p + "mix.right.dt_bias"] = rnd(H * d, std=0.5, mean=-1.0)
            w[p + "mix.right.A_log"] = rnd(H, std=0.5)
            w[p + "mix.right.g1"] = rnd(rg, D, std=D ** -0.5)
            w[p + "mix.right.g2"] = rnd(H * dv, rg, std=rg ** -0.5)
            w[p + "mix.right.norm"] = rnd(dv, std=0.1, mean=1.0)
            w[p + "mix.right.o"] = rnd(D, H * dv, std=(H * dv) ** -0.5)
            w[p + "mix.left.out"] = rnd(D, std=0.1, mean=1.0)
            w[p + "mix.right.out"] = rnd(D, std=0.1, mean=1.0)
        else:
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            for n, rows in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv)):
                w[p + "mix." + n] = rnd(rows, D, std=D ** -0.5)
            w[p + "mix.norm"] = rnd(H * dv, std=0.1, mean=1.0)
            w[p + "mix.o"] = rnd(D, H * dv, std=(H * dv) ** -0.5)
        mlp = spec["mlp"]
        if mlp is not None and mlp["kind"] == "dense":
            w[p + "mlp.up"] = rnd(mlp["ff"], D, std=D ** -0.5)
            w[p + "mlp.down"] = rnd(D, mlp["ff"], std=mlp["ff"] ** -0.5)
        elif mlp is not None:
            E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            w[p + "mlp.router"] = rnd(E, D, std=2.0 * D ** -0.5)
            for e in range(E):
                w[f"{p}mlp.e{e}.gate"] = rnd(ff, D, std=D ** -0.5)
                w[f"{p}mlp.e{e}.up"] = rnd(ff, D, std=D ** -0.5)
                w[f"{p}mlp.e{e}.down"] = rnd(D, ff, std=ff ** -0.5)
    return w


def row_errors(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Per row: rms over the vocabulary of the difference (means taken off) over the rms of the expected row."""
    d = got.double().cpu() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want.double() - want.double().mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-9)


def within(errors: torch.Tensor, tol: float, sixteen: bool) -> bool:
    """fp32: every row within tol.  16-bit: every row within 3 tol and all but one in fifty within tol -- a head's output
    that happens to be near zero (a first token whose query and key are nearly orthogonal, say) is divided by its own root
    mean square, which turns the rounding of 16-bit projections into a change of direction at that one place."""
    if not sixteen:
        return bool(errors.max() < tol)
    return bool(errors.max() < 3 * tol) and int((errors >= tol).sum()) <= max(1, errors.numel() // 50)


def replay_and_compare(runner, cfg, weights, prompts, schedule, tol, want_all=None):
    """schedule: list of steps, each a list of (request name, token count).  Every token's logits are asked for and
    compared with the oracle's logits of the whole prompt; a request ends with its last token.  Returns the worst error."""
    sixteen = runner.dtype != torch.float32
    errors = []
    from sglang_custom_amd.managers.trace_replay import TraceReplayer

    rp = TraceReplayer(runner)
    want = want_all if want_all is not None else {k: ref.forward(public(cfg), weights, p) for k, p in prompts.items()}
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
