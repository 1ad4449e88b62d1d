"""Gatarax: a decoder-only model on an fp32 residual stream whose layers run their mixer and their feed-forward in
parallel off ONE pre-norm, x <- x + mixer(h + C1(h)) + ff(h + C2(h)) with h = N(x) (1 + w) and C1, C2 short causal
convolutions over time.  The mixer is, layer by layer, either a pair of branches side by side -- softmax attention over a
sliding window with a sink in the denominator, and a gated delta rule with a decay per key channel, each output
RMS-normed over the model width, half their sum taken -- or a linear recurrence with one fixed decay per head
("lightning").  The feed-forward is squared-ReLU dense or a mixture of SiLU-gated experts chosen by softmax scores within
the best groups.  The output head is the embedding table.  (No counterpart in the reference; the module layout follows its
model files, python/sglang/srt/models/deepseek_v2.py for the mixture.)

Per layer (T tokens, width D), besides the GEMMs' own launches:

  OffsetRMSNorm            h = N(x) (1 + w), fp32 in, activation dtype out                                   1 launch
  ShortCausalConv          (h + C1(h), h + C2(h)): two filters over one input                                1 launch (+ 1 state)
  parallel   in_proj: [left q | k | v | right q | k | v | beta | a1 | g1] in one GEMM (the left part with its biases)
             left    ShortCausalConv on q | k | v; k and v into the cache; WindowSinkAttention; o (with bias)
             right   ShortCausalConv + silu on q | k | v; unit vectors of q | k in fp32 (one launch); a2(a1) -> fp32 decay
                     logits; GatedDeltaRule; g2(g1); HeadNormGate (sigmoid); o
  lightning  in_proj: [q | k | v | g]; silu on q | k | v; LinearRecurrence (fixed decays); HeadNormGate over all heads
             at once (sigmoid); o
  ff         dense: up, squared relu, down            moe: fp32 router logits, route, align, two grouped GEMMs, silu * up
  BranchResidualAdd        x += 0.5 (N(left) w_l + N(right) w_r) + ff   (or  x += mixer + ff), the experts' weighted sum
                           taken inside                                                                     1 launch, fp32

Norms, attention scores / weights, decays and everything else that enters a recurrence after the projections and
convolutions, recurrent state, router and the residual sum are fp32 in every dtype; `dtype` is what the projections and
convolutions read and write.  Every size comes from the configuration, layer by layer.  Tensor parallelism is not
implemented for this family (its head counts need not divide)."""
from typing import Dict

import torch
from torch import nn

from ..distributed.parallel_state import get_tensor_model_parallel_world_size
from ..layers.activation import Activation
from ..layers.linear import ReplicatedLinear
from ..layers.linear_recurrence import GatedDeltaRule, HeadNormGate, HeadNormRope, LinearRecurrence
from ..layers.logits_processor import LogitsProcessor
from ..layers.moe import GroupedExperts, GroupedTopKRouter
from ..layers.pre_norm import BranchResidualAdd, OffsetRMSNorm
from ..layers.short_conv import ShortCausalConv
from ..layers.vocab_parallel_embedding import ParallelLMHead
from ..layers.window_attention import WindowSinkAttention
from ..ops_backend import get_ops

UNIT_EPS = 1e-6            # inside the root of the unit-vector norm of the delta rule's q and k: x / sqrt(sum x^2 + 1e-6)
DEFAULT_LOW_RANK = 16      # rank of the decay and gate projections of a delta-rule branch built without a checkpoint


class GataraxParallelMixer(nn.Module):
    """Windowed attention with a sink (left) beside a gated delta rule (right); both read the same rows."""

    def __init__(self, hidden: int, mx: dict, eps: float, layer_id: int, dtype, device, decay_rank: int, gate_rank: int):
        super().__init__()
        lf, rt = mx["left"], mx["right"]
        self.lH, self.lG, self.ld, self.ldv = lf["heads"], lf.get("kv_heads", lf["heads"]), lf["dim"], lf.get("vdim", lf["dim"])
        self.rH, self.rG, self.rd, self.rdv = rt["heads"], rt.get("kv_heads", rt["heads"]), rt["dim"], rt["vdim"]
        self.decay_rank, self.gate_rank = decay_rank, gate_rank
        self.left_width = (self.lH + self.lG) * self.ld + self.lG * self.ldv
        self.right_width = 2 * self.rG * self.rd + self.rH * self.rdv
        out = self.left_width + self.right_width + self.rH + decay_rank + gate_rank
        self.in_proj = ReplicatedLinear(hidden, out, dtype, device)
        # the left projections have biases; the other columns' entries stay zero
        self.in_bias = nn.Parameter(torch.zeros(out, dtype=dtype, device=device), requires_grad=False)
        # left: convolution on [q | k | v], keys and values to the cache, attention, output projection with bias
        self.left_conv = ShortCausalConv(self.left_width, lf["conv"], (layer_id, "left"), dtype, device)
        self.attn = WindowSinkAttention(self.lH, self.lG, self.ld, self.ldv, lf["scale"], lf["mask"]["size"], layer_id, device)
        self.left_o = ReplicatedLinear(self.lH * self.ldv, hidden, dtype, device)
        self.left_o_bias = nn.Parameter(torch.zeros(hidden, dtype=dtype, device=device), requires_grad=False)
        # right: convolution + silu on [q | k | v], unit vectors, decay logits, delta rule, normed and gated read-out
        self.right_conv = ShortCausalConv(self.right_width, rt["conv"], (layer_id, "right"), dtype, device, act="silu")
        # x / sqrt(sum x^2 + e) = x / sqrt(d) / sqrt(mean x^2 + e / d): the head norm with a unit weight does it
        d = self.rd
        # (q and k lie side by side: one launch; q's further factor d^-1/2 rides in the rule's q_scale)
        self.qk_unit = HeadNormRope(d, 0, 1.0, True, UNIT_EPS / d, dtype, device, with_norm=True, scale=d ** -0.5)
        self.a2 = ReplicatedLinear(decay_rank, self.rH * d, dtype, device)
        self.g2 = ReplicatedLinear(gate_rank, self.rH * self.rdv, dtype, device)
        self.rule = GatedDeltaRule(self.rH, self.rG, d, self.rdv, layer_id, device, q_scale=d ** -0.5)
        self.norm_gate = HeadNormGate(self.rdv, eps, dtype, device, with_weight=True, gate_act="sigmoid")
        self.right_o = ReplicatedLinear(self.rH * self.rdv, hidden, dtype, device)

    def forward(self, positions, h, forward_batch):
        ops = get_ops()
        T = h.shape[0]
        p = self.in_proj.quant_method.apply(self.in_proj, h, self.in_bias.data)
        lw, rw = self.left_width, self.right_width
        # ---- left
        c = self.left_conv(p[:, :lw], forward_batch)
        nq, nk = self.lH * self.ld, self.lG * self.ld
        k_cache, v_cache = forward_batch.token_to_kv_pool.get_kv_buffer(self.attn.layer_id)
        ops.set_kv_buffer(k_cache, v_cache, forward_batch.out_cache_loc, c[:, nq: nq + nk], c[:, nq + nk:])      # both in one launch
        o = torch.empty((T, self.lH, self.ldv), dtype=h.dtype, device=h.device)
        self.attn(c[:, :nq].view(T, self.lH, self.ld), forward_batch, o)
        left = self.left_o.quant_method.apply(self.left_o, o.view(T, self.lH * self.ldv), self.left_o_bias.data)
        # ---- right
        r = self.right_conv(p[:, lw: lw + rw], forward_batch)
        gk = self.rG * self.rd
        qk = self.qk_unit(r[:, : 2 * gk].view(T, 2 * self.rG, self.rd), positions, torch.float32)
        q, k = qk[:, : self.rG], qk[:, self.rG:]
        v = r[:, 2 * gk:].view(T, self.rH, self.rdv)
        at = lw + rw
        beta = p[:, at: at + self.rH]
        a1 = p[:, at + self.rH: at + self.rH + self.decay_rank]
        g1 = p[:, at + self.rH + self.decay_rank:]
        z = ops.linear(a1, self.a2.weight.data, out_dtype=torch.float32)       # decay logits, fp32 from here on
        s = self.rule(q, k, v, beta, z, forward_batch)
        right = self.right_o(self.norm_gate(s, self.g2(g1)[0]))[0]
        return left, right


class GataraxLightningMixer(nn.Module):
    def __init__(self, hidden: int, mx: dict, eps: float, layer_id: int, dtype, device):
        super().__init__()
        H, d, dv = mx["heads"], mx["dim"], mx["vdim"]
        self.H, self.d, self.dv = H, d, dv
        self.in_proj = ReplicatedLinear(hidden, 2 * H * d + 2 * H * dv, dtype, device)     # [q | k | v | g]
        self.act = Activation("silu")
        self.recurrence = LinearRecurrence(H, d, dv, layer_id, device, head_decay=mx["decay"])
        # one norm over all heads together: the read-out counts as a single head of width H * dv
        self.norm_gate = HeadNormGate(H * dv, eps, dtype, device, with_weight=True, gate_act="sigmoid")
        self.o_proj = ReplicatedLinear(H * dv, hidden, dtype, device)

    def forward(self, positions, h, forward_batch):
        T, H, d, dv = h.shape[0], self.H, self.d, self.dv
        p = self.in_proj(h)[0]
        n = 2 * H * d + H * dv
        a = self.act(p[:, :n])
        q = a[:, : H * d].view(T, H, d)
        k = a[:, H * d: 2 * H * d].view(T, H, d)
        v = a[:, 2 * H * d:].view(T, H, dv)
        o = self.recurrence(q, k, v, forward_batch)
        return self.o_proj(self.norm_gate(o.view(T, 1, H * dv), p[:, n:]))[0]


class GataraxDenseMLP(nn.Module):
    def __init__(self, hidden: int, ff: int, dtype, device):
        super().__init__()
        self.up = ReplicatedLinear(hidden, ff, dtype, device)
        self.act = Activation("relu2")
        self.down = ReplicatedLinear(ff, hidden, dtype, device)

    def forward(self, h):
        return self.down(self.act(self.up(h)[0]))[0]


class GataraxMoE(nn.Module):
    def __init__(self, hidden: int, mlp: dict, dtype, device):
        super().__init__()
        r = mlp["router"]
        groups = r.get("groups") or {"count": 1, "keep": 1}
        self.router = GroupedTopKRouter(hidden, r["experts"], r["top"], groups["count"], groups["keep"], 1.0, device,
                                        score_fn="softmax", group_best=1, renorm=False, with_correction=False)
        self.experts = GroupedExperts(hidden, mlp["expert"]["ff"], r["experts"], dtype, device, activation="silu_gated")

    def forward(self, h):
        """h: the feed-forward's input; the router reads it widened to fp32."""
        ids, weights = self.router(h if h.dtype == torch.float32 else h.float())
        y, rows = self.experts(h, ids)
        return y, rows, weights


class GataraxDecoderLayer(nn.Module):
    def __init__(self, config, layer_id: int, dtype, device, decay_rank: int, gate_rank: int):
        super().__init__()
        spec = config.layer_specs[layer_id]
        D, eps = config.hidden_size, config.rms_norm_eps
        self.kind = spec["type"]
        mlp = spec.get("mlp")
        self.norm1 = OffsetRMSNorm(D, eps, dtype, device)
        # one launch serves the mixer's and the feed-forward's input convolution: both read the same normed rows
        self.canon = (ShortCausalConv(D, config.canon_taps, (layer_id, "canon"), dtype, device, residual=True, second=mlp is not None)
                      if config.canon_taps else None)
        if self.kind == "parallel":
            self.mixer = GataraxParallelMixer(D, spec["mixer"], eps, layer_id, dtype, device, decay_rank, gate_rank)
            self.add = BranchResidualAdd(D, eps, dtype, device, normed_branches=2, scale=0.5)
        else:
            self.mixer = GataraxLightningMixer(D, spec["mixer"], eps, layer_id, dtype, device)
            self.add = BranchResidualAdd(D, eps, dtype, device, normed_branches=0)
        self.mlp = None
        self.moe = None
        if mlp is not None and mlp["kind"] == "dense":
            self.mlp = GataraxDenseMLP(D, mlp["ff"], dtype, device)
        elif mlp is not None:
            self.moe = GataraxMoE(D, mlp, dtype, device)

    def forward(self, positions, x, forward_batch):
        h = self.norm1(x)
        hm = hf = h
        if self.canon is not None:
            if self.canon.weight2 is not None:
                hm, hf = self.canon(h, forward_batch)
            else:
                hm = self.canon(h, forward_batch)
        if self.kind == "parallel":
            a, b = self.mixer(positions, hm, forward_batch)
        else:
            a, b = self.mixer(positions, hm, forward_batch), None
        if self.mlp is not None:
            self.add(x, a, b, f=self.mlp(hf))
        elif self.moe is not None:
            y, rows, weights = self.moe(hf)
            self.add(x, a, b, f=y, rows=rows, coef=weights)
        else:
            self.add(x, a, b)
        return x


class GataraxModel(nn.Module):
    def __init__(self, config, dtype, device, decay_ranks=None, gate_ranks=None):
        super().__init__()
        D = config.hidden_size
        self.embed_scale = float(config.embedding_scale)
        self.embed = nn.Parameter(torch.zeros(config.vocab_size, D, dtype=dtype, device=device), requires_grad=False)
        self.layers = nn.ModuleList([GataraxDecoderLayer(config, i, dtype, device, (decay_ranks or {}).get(i, DEFAULT_LOW_RANK),
                                                         (gate_ranks or {}).get(i, DEFAULT_LOW_RANK))
                                     for i in range(config.num_hidden_layers)])
        self.norm = OffsetRMSNorm(D, config.rms_norm_eps, dtype, device)
        self.capture_streams = None     # a list here receives the fp32 residual after every layer (tests, debugging)

    def forward(self, input_ids, positions, forward_batch):
        x = get_ops().embedding(input_ids, self.embed.data).float()
        if self.embed_scale != 1.0:
            x.mul_(self.embed_scale)
        for layer in self.layers:
            layer(positions, x, forward_batch)
            if self.capture_streams is not None:
                self.capture_streams.append(x.clone())
        return self.norm(x)


class GataraxForCausalLM(nn.Module):
    needs_sequence_state = True
    supports_hip_graph = False    # a captured decode step pads the batch with row 0 of the request table, whose state slot it would overwrite

    def __init__(self, config, dtype=torch.bfloat16, device="cuda", quant_method_factory=None):
        super().__init__()
        if quant_method_factory is not None:
            raise NotImplementedError("Gatarax runs unquantised (its norms, router, decays and residual are fp32 by design)")
        if get_tensor_model_parallel_world_size() != 1:
            raise NotImplementedError("Gatarax: tensor parallelism is not implemented")
        self.config = config
        self.dtype = dtype
        # built by load_weights / init_random_weights: the ranks of a delta-rule branch's decay and gate projections are
        # read off the checkpoint's tensors
        self.model = None
        self._device = device
        self.lm_head = ParallelLMHead(config.vocab_size, config.hidden_size, dtype, device)
        self.logits_processor = LogitsProcessor(config, logit_scale=config.logit_scale if config.logit_scale != 1.0 else None)

    def _build(self, decay_ranks=None, gate_ranks=None):
        self.model = GataraxModel(self.config, self.dtype, self._device, decay_ranks, gate_ranks)
        self.to(self._device)
        self.lm_head.weight = self.model.embed     # the output head is the embedding table itself

    def sequence_state_spec(self) -> dict:
        cfg = self.config
        convs = {}
        for i, layer in enumerate(self.model.layers):
            if layer.canon is not None:
                convs[(i, "canon")] = (layer.canon.taps, cfg.hidden_size)
            if layer.kind == "parallel":
                convs[(i, "left")] = (layer.mixer.left_conv.taps, layer.mixer.left_width)
                convs[(i, "right")] = (layer.mixer.right_conv.taps, layer.mixer.right_width)
        return dict(layer_num=0, hidden=cfg.hidden_size, matrices=dict(enumerate(cfg.recurrent_layer_shapes)), convs=convs)

    @torch.no_grad()
    def forward(self, input_ids, positions, forward_batch):
        hidden_states = self.model(input_ids, positions, forward_batch)
        return self.logits_processor(input_ids, hidden_states, self.lm_head, forward_batch)

    def _linears(self):
        for layer in self.model.layers:
            mx = layer.mixer
            if layer.kind == "parallel":
                yield from (mx.in_proj, mx.left_o, mx.a2, mx.g2, mx.right_o)
            else:
                yield from (mx.in_proj, mx.o_proj)
            if layer.mlp is not None:
                yield from (layer.mlp.up, layer.mlp.down)

    @torch.no_grad()
    def load_weights(self, weights: Dict[str, torch.Tensor]) -> None:
        """Checkpoint names: embed, final.norm, l<i>.norm1, l<i>.canon1, l<i>.canon2; a parallel mixer's
        l<i>.mix.left.{q, k, v, o} with .b biases and {q, k, v}.conv, l<i>.mix.right.{q, k, v} with .conv,
        l<i>.mix.right.{b, a1, a2, dt_bias, A_log, g1, g2, norm, o}, l<i>.mix.{left, right}.out; a lightning mixer's
        l<i>.mix.{q, k, v, g, o, norm}; l<i>.mlp.{up, down} or l<i>.mlp.{router, e<j>.gate, e<j>.up, e<j>.down}; linear
        weights [out, in].  Projections that read the same rows are stacked, the experts' weights are stacked per layer."""
        cfg = self.config
        par = [i for i, s in enumerate(cfg.layer_specs) if s["type"] == "parallel"]
        self._build(decay_ranks={i: int(weights[f"l{i}.mix.right.a1"].shape[0]) for i in par},
                    gate_ranks={i: int(weights[f"l{i}.mix.right.g1"].shape[0]) for i in par})

        def put(param, value):
            assert tuple(param.shape) == tuple(value.shape), f"shape {tuple(value.shape)} for a parameter {tuple(param.shape)}"
            param.data.copy_(value.to(dtype=param.dtype), non_blocking=True)

        m = self.model
        put(m.embed, weights["embed"])
        put(m.norm.weight, weights["final.norm"])
        for i, layer in enumerate(m.layers):
            p, mx = f"l{i}.", layer.mixer
            put(layer.norm1.weight, weights[p + "norm1"])
            if layer.canon is not None:
                put(layer.canon.weight, weights[p + "canon1"])
                if layer.canon.weight2 is not None:
                    put(layer.canon.weight2, weights[p + "canon2"])
            if layer.kind == "parallel":
                lf, rt = p + "mix.left.", p + "mix.right."
                put(mx.in_proj.weight, torch.cat([weights[lf + n] for n in ("q", "k", "v")]
                                                 + [weights[rt + n] for n in ("q", "k", "v", "b", "a1", "g1")], 0))
                bias = torch.cat([weights[lf + n + ".b"] for n in ("q", "k", "v")], 0)
                mx.in_bias.data.zero_()
                mx.in_bias.data[: bias.numel()].copy_(bias.to(mx.in_bias.dtype))
                put(mx.left_conv.weight, torch.cat([weights[lf + n + ".conv"] for n in ("q", "k", "v")], 0))
                put(mx.left_o.weight, weights[lf + "o"])
                put(mx.left_o_bias, weights[lf + "o.b"])
                put(mx.right_conv.weight, torch.cat([weights[rt + n + ".conv"] for n in ("q", "k", "v")], 0))
                put(mx.a2.weight, weights[rt + "a2"])
                put(mx.g2.weight, weights[rt + "g2"])
                put(mx.rule.rate_bias, weights[rt + "dt_bias"])
                put(mx.rule.rate_log, weights[rt + "A_log"])
                put(mx.norm_gate.weight, weights[rt + "norm"])
                put(mx.right_o.weight, weights[rt + "o"])
                put(layer.add.weight_a, weights[lf + "out"])
                put(layer.add.weight_b, weights[rt + "out"])
            else:
                put(mx.in_proj.weight, torch.cat([weights[p + "mix." + n] for n in ("q", "k", "v", "g")], 0))
                put(mx.norm_gate.weight, weights[p + "mix.norm"])
                put(mx.o_proj.weight, weights[p + "mix.o"])
            if layer.mlp is not None:
                put(layer.mlp.up.weight, weights[p + "mlp.up"])
                put(layer.mlp.down.weight, weights[p + "mlp.down"])
            if layer.moe is not None:
                E = layer.moe.router.num_experts
                put(layer.moe.router.weight, weights[p + "mlp.router"])
                put(layer.moe.experts.w_up, torch.stack([torch.cat([weights[f"{p}mlp.e{e}.gate"], weights[f"{p}mlp.e{e}.up"]], 0)
                                                         for e in range(E)]))
                put(layer.moe.experts.w_down, torch.stack([weights[f"{p}mlp.e{e}.down"] for e in range(E)]))
        self.process_weights_after_loading()

    def process_weights_after_loading(self) -> None:
        for lin in self._linears():
            lin.quant_method.process_weights_after_loading(lin)

    @torch.no_grad()
    def init_random_weights(self, seed: int = 0, std: float = 0.02) -> None:
        if self.model is None:
            # without a checkpoint the low ranks are the configuration's optional "decay_rank" / "gate_rank", or the default
            par = {i: s["mixer"]["right"] for i, s in enumerate(self.config.layer_specs) if s["type"] == "parallel"}
            self._build(decay_ranks={i: int(r["decay_rank"]) for i, r in par.items() if r.get("decay_rank")},
                        gate_ranks={i: int(r["gate_rank"]) for i, r in par.items() if r.get("gate_rank")})
        dev = self.lm_head.weight.device
        g = torch.Generator(device=dev).manual_seed(seed)
        for name, p in self.named_parameters():
            w = torch.randn(p.shape, generator=g, device=p.device, dtype=torch.float32)
            if name.endswith("norm1.weight") or name.endswith("model.norm.weight"):
                p.data.copy_((0.1 * w).to(p.dtype))                      # stored around zero
            elif name.endswith("norm_gate.weight") or name.endswith("add.weight_a") or name.endswith("add.weight_b"):
                p.data.copy_((1.0 + 0.1 * w).to(p.dtype))
            elif name.endswith("attn.sink"):
                p.data.zero_()
            elif name.endswith("rate_log") or name.endswith("rate_bias") or name.endswith("in_bias") or name.endswith("left_o_bias"):
                p.data.copy_((0.1 * w).to(p.dtype))
            elif name.endswith("canon.weight") or name.endswith("canon.weight2") or name.endswith("conv.weight"):
                p.data.copy_((w * p.shape[-1] ** -0.5).to(p.dtype))
            elif name.endswith("qk_unit.weight"):
                p.data.fill_(1.0)
            elif name.endswith("embed"):
                p.data.copy_((w / max(self.model.embed_scale, 1e-6)).to(p.dtype))
            else:
                p.data.copy_((w * (std if p.dim() < 2 else p.shape[-1] ** -0.5)).to(p.dtype))
        for layer in self.model.layers:
            if layer.kind == "parallel":
                layer.mixer.in_bias.data[layer.mixer.left_width:].zero_()      # only the left projections have biases
        self.process_weights_after_loading()
