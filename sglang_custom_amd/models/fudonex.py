"""Fudonex: a decoder-only model on an fp32 residual stream whose sublayers read the stream itself and are normed on
their OUTPUT: x <- x + m * l1 * N(mixer(x)) (1 + w1), then x <- x + m * l2 * N(ff(x)) (1 + w2), with N the RMS norm, the
weights stored around zero, l1 / l2 per-channel layer scales and m one configured factor.  The mixer is, layer by layer,

  attention   softmax attention with grouped key heads over the last W tokens and, before them, one averaged key / value per
              complete block of P tokens; biased projections, an RMS norm with a shared weight on every query and key head,
              a rotation of the first features of each head in the half-split pairing with frequencies stretched for long
              sequences, values divided by their root mean square, a sink logit per head in the denominator, a sigmoid gate
              per head on the result.  A layer may read another layer's cached keys and values instead of making its own.
  mamba2      a state-space recurrence: one projection gives [z | x | B | C | dt]; x | B | C pass a short causal convolution
              with bias and SiLU; dt = softplus(dt + bias); per head S <- exp(-exp(A) dt) S + dt B x^T, y = S^T C + D x; then
              y * silu(z), an RMS norm in equal parts, the output projection.
  delta       the gated delta rule with one decay per head and token: q, k, v through short causal convolutions and SiLU,
              q and k made unit vectors, beta = sigmoid, S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q; then a
              norm per head times silu(gate), the output projection.

The feed-forward is SiLU-gated dense, or absent.  The output head is the embedding table; the logits are capped by a tanh.
(No counterpart in the reference; the module layout follows its model files, python/sglang/srt/models/llama.py.)

Per layer (T tokens, width D), besides the GEMMs' own launches:

  attention   in_proj [q | k | v | g] with its biases (a layer that borrows its keys: [q | g]); QKVHeadNormRope: q normed and
              rotated, k the same straight into the cache, the values' unit norm straight into the cache, one launch
              (HeadNormRope on q alone in a borrowing layer); the averages of the blocks the step completes;
              WindowSinkAttention (gate inside); o
  mamba2      in_proj [z | x | B | C] and, in fp32, dt; ShortCausalConv (bias, silu); StateSpaceRecurrence; GatedGroupNorm; o
  delta       in_proj [q | k | v | g] and, in fp32, [beta | a]; ShortCausalConv (silu); unit vectors of q | k (one launch);
              GatedDeltaRule (decay per head); HeadNormGate; o
  NormedResidualAdd   x += m * l * N(y) (1 + w) in place, which also writes the activation-dtype copy of x that the next
                      sublayer's projections read                                                         1 launch, fp32
  ff          gate_up, silu * up, down

Norms, positions and angles, attention scores / weights, step sizes, decays and everything else that enters a recurrence
after the projections and convolutions, recurrent state and the residual sum are fp32 in every dtype; `dtype` is what the
projections and convolutions read and write.  Every size comes from the configuration, layer by layer.  Tensor
parallelism is not implemented for this family (its head counts need not divide)."""
from typing import Dict, Optional

import torch
from torch import nn

from ..distributed.parallel_state import get_tensor_model_parallel_world_size
from ..layers.activation import SiluAndMul
from ..layers.linear import ReplicatedLinear
from ..layers.linear_recurrence import (
    GatedDeltaRule,
    GatedGroupNorm,
    HeadNormGate,
    HeadNormRope,
    QKVHeadNormRope,
    StateSpaceRecurrence,
)
from ..layers.logits_processor import LogitsProcessor
from ..layers.post_norm import NormedResidualAdd
from ..layers.pre_norm import OffsetRMSNorm
from ..layers.rotary_embedding import scaled_pair_inv_freq
from ..layers.short_conv import ShortCausalConv
from ..layers.vocab_parallel_embedding import ParallelLMHead
from ..layers.window_attention import WindowSinkAttention
from ..ops_backend import get_ops

UNIT_EPS = 1e-6            # inside the root of the unit-vector norm of the delta rule's q and k: x / sqrt(sum x^2 + 1e-6)


class FudonexAttention(nn.Module):
    def __init__(self, hidden: int, mx: dict, eps: float, layer_id: int, dtype, device, store_pools=()):
        """store_pools: the block lengths whose averages this layer writes after its cache write: its own mask's and those of
        the layers that read its cache."""
        super().__init__()
        H, G, d = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"]
        dv = mx.get("vdim", d)
        self.H, self.G, self.d, self.dv = H, G, d, dv
        self.kv_from: Optional[int] = mx.get("kv_from")
        rot = mx.get("rot") or {}
        rot_dims = int(rot.get("dims", 0))
        freqs, mag = scaled_pair_inv_freq(rot["base"], rot_dims, rot.get("scaling")) if rot_dims else (None, 1.0)
        mask = mx.get("mask") or {}
        own = self.kv_from is None
        self.q_width, self.k_width, self.v_width = H * d, (G * d if own else 0), (G * dv if own else 0)
        out = self.q_width + self.k_width + self.v_width + H                       # [q | k | v | g]
        self.in_proj = ReplicatedLinear(hidden, out, dtype, device)
        # q, k and v have biases; the gate's entries stay zero
        self.in_bias = nn.Parameter(torch.zeros(out, dtype=dtype, device=device), requires_grad=False)
        if own:
            # q and k normed and rotated, v divided by its root mean square, k and v into the cache: one launch
            self.qkv_norm = QKVHeadNormRope(d, dv, rot_dims, 1.0, False, eps, dtype, device, inv_freq=freqs, rot_mag=mag)
        else:
            self.q_norm = HeadNormRope(d, rot_dims, 1.0, False, eps, dtype, device, with_norm=True, inv_freq=freqs, rot_mag=mag)
        self.attn = WindowSinkAttention(H, G, d, dv, mx["scale"], int(mask.get("size", 0)), layer_id, device,
                                        pool=int(mask.get("pool", 0) or 0), kv_layer_id=self.kv_from,
                                        store_pools=tuple(store_pools) if own else ())
        self.o_proj = ReplicatedLinear(H * dv, hidden, dtype, device)

    def forward(self, positions, h, forward_batch):
        T, H, G, d, dv = h.shape[0], self.H, self.G, self.d, self.dv
        p = self.in_proj.quant_method.apply(self.in_proj, h, self.in_bias.data)
        if self.kv_from is None:
            k_cache, v_cache = forward_batch.token_to_kv_pool.get_kv_buffer(self.attn.layer_id)
            kq = self.q_width
            q = self.qkv_norm(p[:, :kq].view(T, H, d), p[:, kq: kq + self.k_width].view(T, G, d),
                              p[:, kq + self.k_width: kq + self.k_width + self.v_width].view(T, G, dv), positions, k_cache, v_cache,
                              forward_batch.out_cache_loc)
            self.attn.store_blocks(forward_batch)
        else:
            q = self.q_norm(p[:, : self.q_width].view(T, H, d), positions, h.dtype)
        o = torch.empty((T, H, dv), dtype=h.dtype, device=h.device)
        self.attn(q, forward_batch, o, head_gate=p[:, self.q_width + self.k_width + self.v_width:])
        return self.o_proj(o.view(T, H * dv))[0]


class FudonexStateSpace(nn.Module):
    def __init__(self, hidden: int, mx: dict, eps: float, layer_id: int, dtype, device):
        super().__init__()
        H, dv, N, G = mx["heads"], mx["vdim"], mx["state"], mx.get("groups", 1)
        self.H, self.dv, self.N, self.G = H, dv, N, G
        self.inner = H * dv
        self.conv_width = self.inner + 2 * G * N
        self.in_proj = ReplicatedLinear(hidden, self.inner + self.conv_width, dtype, device)        # [z | x | B | C]
        self.dt_proj = ReplicatedLinear(hidden, H, dtype, device)                                     # step-size logits, fp32 out
        self.conv = ShortCausalConv(self.conv_width, mx["conv"], (layer_id, "ssm"), dtype, device, act="silu", bias=True)
        self.recurrence = StateSpaceRecurrence(H, G, N, dv, layer_id, device)
        self.norm = GatedGroupNorm(self.inner, int(mx.get("norm_groups", 1)), eps, dtype, device)
        self.o_proj = ReplicatedLinear(self.inner, hidden, dtype, device)

    def forward(self, positions, h, forward_batch):
        T, H, dv, N, G = h.shape[0], self.H, self.dv, self.N, self.G
        p = self.in_proj(h)[0]
        dt = get_ops().linear(h, self.dt_proj.weight.data, out_dtype=torch.float32)
        c = self.conv(p[:, self.inner:], forward_batch)
        x = c[:, : self.inner].view(T, H, dv)
        B = c[:, self.inner: self.inner + G * N].view(T, G, N)
        C = c[:, self.inner + G * N:].view(T, G, N)
        y = self.recurrence(C, B, x, dt, forward_batch)
        return self.o_proj(self.norm(y.view(T, self.inner), p[:, : self.inner]))[0]


class FudonexDeltaRule(nn.Module):
    def __init__(self, hidden: int, mx: dict, eps: float, layer_id: int, dtype, device):
        super().__init__()
        H, G, d, dv = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx["vdim"]
        self.H, self.G, self.d, self.dv = H, G, d, dv
        self.conv_width = 2 * G * d + H * dv
        self.in_proj = ReplicatedLinear(hidden, self.conv_width + H * dv, dtype, device)            # [q | k | v | g]
        self.ba_proj = ReplicatedLinear(hidden, 2 * H, dtype, device)                                 # [beta | a] logits, fp32 out
        self.conv = ShortCausalConv(self.conv_width, mx["conv"], (layer_id, "delta"), dtype, device, act="silu")
        # x / sqrt(sum x^2 + e) = x / sqrt(d) / sqrt(mean x^2 + e / d): the head norm with a unit weight does it; q and k lie
        # side by side (one launch), q's further factor d^-1/2 rides in the rule's q_scale
        self.qk_unit = HeadNormRope(d, 0, 1.0, False, UNIT_EPS / d, dtype, device, with_norm=True, scale=d ** -0.5)
        self.rule = GatedDeltaRule(H, G, d, dv, layer_id, device, q_scale=d ** -0.5, decay_per_head=True)
        self.norm_gate = HeadNormGate(dv, eps, dtype, device, with_weight=True, gate_act="silu")
        self.o_proj = ReplicatedLinear(H * dv, hidden, dtype, device)

    def forward(self, positions, h, forward_batch):
        T, H, G, d, dv = h.shape[0], self.H, self.G, self.d, self.dv
        p = self.in_proj(h)[0]
        ba = get_ops().linear(h, self.ba_proj.weight.data, out_dtype=torch.float32)
        c = self.conv(p[:, : self.conv_width], forward_batch)
        qk = self.qk_unit(c[:, : 2 * G * d].view(T, 2 * G, d), positions, torch.float32)
        v = c[:, 2 * G * d:].view(T, H, dv)
        s = self.rule(qk[:, :G], qk[:, G:], v, ba[:, :H], ba[:, H:], forward_batch)
        return self.o_proj(self.norm_gate(s, p[:, self.conv_width:]))[0]


class FudonexMLP(nn.Module):
    def __init__(self, hidden: int, ff: int, dtype, device):
        super().__init__()
        self.gate_up = ReplicatedLinear(hidden, 2 * ff, dtype, device)
        self.act = SiluAndMul()
        self.down = ReplicatedLinear(ff, hidden, dtype, device)

    def forward(self, h):
        return self.down(self.act(self.gate_up(h)[0]))[0]


_MIXERS = {"attention": FudonexAttention, "mamba2": FudonexStateSpace, "delta": FudonexDeltaRule}


class FudonexDecoderLayer(nn.Module):
    def __init__(self, config, layer_id: int, dtype, device):
        super().__init__()
        spec = config.layer_specs[layer_id]
        D, eps, m = config.hidden_size, config.rms_norm_eps, config.residual_mult
        self.kind = spec["type"]
        extra = dict(store_pools=config.kv_layer_pools[layer_id]) if self.kind == "attention" else {}
        self.mixer = _MIXERS[self.kind](D, spec["mixer"], eps, layer_id, dtype, device, **extra)
        self.add1 = NormedResidualAdd(D, eps, dtype, device, offset=1.0, mult=m, layer_scale=True)
        self.mlp = None
        if spec.get("mlp") is not None:
            self.mlp = FudonexMLP(D, spec["mlp"]["ff"], dtype, device)
            self.add2 = NormedResidualAdd(D, eps, dtype, device, offset=1.0, mult=m, layer_scale=True)

    def forward(self, positions, x, h, forward_batch):
        """x: the fp32 stream, updated in place; h: its copy in the activation dtype.  Returns the new h."""
        h = self.add1(x, self.mixer(positions, h, forward_batch))
        if self.mlp is not None:
            h = self.add2(x, self.mlp(h))
        return h


class FudonexModel(nn.Module):
    def __init__(self, config, dtype, device):
        super().__init__()
        D = config.hidden_size
        self.dtype = dtype
        self.embed_scale = float(config.embedding_scale)
        self.embed = nn.Parameter(torch.zeros(config.vocab_size, D, dtype=dtype, device=device), requires_grad=False)
        self.layers = nn.ModuleList([FudonexDecoderLayer(config, i, dtype, device) for i in range(config.num_hidden_layers)])
        self.norm = OffsetRMSNorm(D, config.rms_norm_eps, dtype, device)
        self.capture_streams = None     # a list here receives the fp32 residual after every layer (tests, debugging)

    def forward(self, input_ids, positions, forward_batch):
        x = get_ops().embedding(input_ids, self.embed.data).float()
        if self.embed_scale != 1.0:
            x.mul_(self.embed_scale)
        h = x if self.dtype == torch.float32 else x.to(self.dtype)
        for layer in self.layers:
            h = layer(positions, x, h, forward_batch)
            if self.capture_streams is not None:
                self.capture_streams.append(x.clone())
        return self.norm(x)


class FudonexForCausalLM(nn.Module):
    supports_hip_graph = False    # a captured decode step pads the batch with row 0 of the request table, whose state slot it would overwrite

    def __init__(self, config, dtype=torch.bfloat16, device="cuda", quant_method_factory=None):
        super().__init__()
        if quant_method_factory is not None:
            raise NotImplementedError("Fudonex runs unquantised (its norms, decays, step sizes and residual are fp32 by design)")
        if get_tensor_model_parallel_world_size() != 1:
            raise NotImplementedError("Fudonex: tensor parallelism is not implemented")
        self.config = config
        self.dtype = dtype
        self.needs_sequence_state = bool(config.needs_sequence_state)
        self.model = FudonexModel(config, dtype, device)
        self.lm_head = ParallelLMHead(config.vocab_size, config.hidden_size, dtype, device)
        self.to(device)
        self.lm_head.weight = self.model.embed     # the head reads the embedding's parameter; the embedding's factor is not applied on this side
        self.logits_processor = LogitsProcessor(config)

    def sequence_state_spec(self) -> dict:
        cfg = self.config
        convs = {layer.mixer.conv.state_key: (layer.mixer.conv.taps, layer.mixer.conv_width)
                 for layer in self.model.layers if layer.kind != "attention"}
        matrices = {i: s for i, s in enumerate(cfg.recurrent_layer_shapes) if s is not None}
        return dict(layer_num=0, hidden=cfg.hidden_size, matrices=matrices, convs=convs)

    @torch.no_grad()
    def forward(self, input_ids, positions, forward_batch):
        hidden_states = self.model(input_ids, positions, forward_batch)
        return self.logits_processor(input_ids, hidden_states, self.lm_head, forward_batch)

    def _linears(self):
        for layer in self.model.layers:
            mx = layer.mixer
            yield from (mx.in_proj, mx.o_proj)
            if layer.kind == "mamba2":
                yield mx.dt_proj
            elif layer.kind == "delta":
                yield mx.ba_proj
            if layer.mlp is not None:
                yield from (layer.mlp.gate_up, layer.mlp.down)

    @torch.no_grad()
    def load_weights(self, weights: Dict[str, torch.Tensor]) -> None:
        """Checkpoint names: embed, final.norm, l<i>.norm1, l<i>.norm2, l<i>.ls1, l<i>.ls2; an attention mixer's
        l<i>.mix.{q, k, v} with .b biases, {q, k}.norm, sink, g, o (no k, v, k.norm in a layer that borrows its keys); a
        mamba2 mixer's l<i>.mix.{in, conv, conv.b, dt_bias, A_log, D, norm, o}; a delta mixer's l<i>.mix.{q, k, v} with
        .conv, {b, a, dt_bias, A_log, g, norm, o}; l<i>.mlp.{gate, up, down}; linear weights [out, in].  Projections that
        read the same rows are stacked."""

        def put(param, value):
            assert tuple(param.shape) == tuple(value.shape), f"shape {tuple(value.shape)} for a parameter {tuple(param.shape)}"
            param.data.copy_(value.to(dtype=param.dtype), non_blocking=True)

        m = self.model
        put(m.embed, weights["embed"])
        put(m.norm.weight, weights["final.norm"])
        for i, layer in enumerate(m.layers):
            p, mx = f"l{i}.", layer.mixer
            x = p + "mix."
            put(layer.add1.weight, weights[p + "norm1"])
            put(layer.add1.layer_scale, weights[p + "ls1"])
            if layer.kind == "attention":
                names = ("q", "k", "v") if mx.kv_from is None else ("q",)
                put(mx.in_proj.weight, torch.cat([weights[x + n] for n in names] + [weights[x + "g"]], 0))
                bias = torch.cat([weights[x + n + ".b"] for n in names], 0)
                mx.in_bias.data.zero_()
                mx.in_bias.data[: bias.numel()].copy_(bias.to(mx.in_bias.dtype))
                if mx.kv_from is None:
                    put(mx.qkv_norm.q_weight, weights[x + "q.norm"])
                    put(mx.qkv_norm.k_weight, weights[x + "k.norm"])
                else:
                    put(mx.q_norm.weight, weights[x + "q.norm"])
                put(mx.attn.sink, weights[x + "sink"])
            elif layer.kind == "mamba2":
                w_in = weights[x + "in"]
                n = mx.inner + mx.conv_width
                put(mx.in_proj.weight, w_in[:n])
                put(mx.dt_proj.weight, w_in[n:])
                put(mx.conv.weight, weights[x + "conv"])
                put(mx.conv.bias, weights[x + "conv.b"])
                put(mx.recurrence.dt_bias, weights[x + "dt_bias"])
                put(mx.recurrence.rate_log, weights[x + "A_log"])
                put(mx.recurrence.skip, weights[x + "D"])
                put(mx.norm.weight, weights[x + "norm"])
            else:
                put(mx.in_proj.weight, torch.cat([weights[x + n] for n in ("q", "k", "v", "g")], 0))
                put(mx.ba_proj.weight, torch.cat([weights[x + "b"], weights[x + "a"]], 0))
                put(mx.conv.weight, torch.cat([weights[x + n + ".conv"] for n in ("q", "k", "v")], 0))
                put(mx.rule.rate_bias, weights[x + "dt_bias"])
                put(mx.rule.rate_log, weights[x + "A_log"])
                put(mx.norm_gate.weight, weights[x + "norm"])
            put(mx.o_proj.weight, weights[x + "o"])
            if layer.mlp is not None:
                put(layer.add2.weight, weights[p + "norm2"])
                put(layer.add2.layer_scale, weights[p + "ls2"])
                put(layer.mlp.gate_up.weight, torch.cat([weights[p + "mlp.gate"], weights[p + "mlp.up"]], 0))
                put(layer.mlp.down.weight, weights[p + "mlp.down"])
        self.process_weights_after_loading()

    def process_weights_after_loading(self) -> None:
        for lin in self._linears():
            lin.quant_method.process_weights_after_loading(lin)

    @torch.no_grad()
    def init_random_weights(self, seed: int = 0, std: float = 0.02) -> None:
        dev = self.lm_head.weight.device
        g = torch.Generator(device=dev).manual_seed(seed)
        for name, p in self.named_parameters():
            w = torch.randn(p.shape, generator=g, device=p.device, dtype=torch.float32)
            if name.endswith("add1.weight") or name.endswith("add2.weight") or name.endswith("model.norm.weight"):
                p.data.copy_((0.1 * w).to(p.dtype))                      # stored around zero
            elif name.endswith("layer_scale") or name.endswith("q_norm.weight") or name.endswith("q_weight") or name.endswith("k_weight") \
                    or name.endswith("norm_gate.weight") or name.endswith("mixer.norm.weight"):
                p.data.copy_((1.0 + 0.1 * w).to(p.dtype))
            elif name.endswith("qk_unit.weight"):
                p.data.fill_(1.0)
            elif name.endswith("attn.sink") or name.endswith("rate_log") or name.endswith("rate_bias") or name.endswith("dt_bias") \
                    or name.endswith("in_bias") or name.endswith("conv.bias"):
                p.data.copy_((0.1 * w).to(p.dtype))
            elif name.endswith("recurrence.skip"):
                p.data.copy_((1.0 + 0.1 * w).to(p.dtype))
            elif name.endswith("conv.weight"):
                p.data.copy_((w * p.shape[-1] ** -0.5).to(p.dtype))
            elif name.endswith("embed"):
                p.data.copy_((w / max(self.model.embed_scale, 1e-6)).to(p.dtype))
            else:
                p.data.copy_((w * (std if p.dim() < 2 else p.shape[-1] ** -0.5)).to(p.dtype))
        for layer in self.model.layers:
            if layer.kind == "attention":
                layer.mixer.in_bias.data[layer.mixer.in_bias.numel() - layer.mixer.H:].zero_()      # the gate has no bias
        self.process_weights_after_loading()
