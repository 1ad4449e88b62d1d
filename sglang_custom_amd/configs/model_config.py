"""ModelConfig: head / KV geometry the hot path needs (the fields of the reference's
python/sglang/srt/configs/model_config.py that model_runner, the pools and the attention
backend read), built from a HuggingFace-style config dict or config.json."""
import json
import os
from types import SimpleNamespace
from typing import Optional

import torch

_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16,
           "half": torch.float16, "auto": None}


class ModelConfig:
    def __init__(self, hf_config: dict, dtype: str = "auto", context_length: Optional[int] = None,
                 quantization: Optional[str] = None):
        c = dict(hf_config)
        self.hf_config = SimpleNamespace(**c)
        self.architecture = c.get("architecture") or (c.get("architectures") or ["LlamaForCausalLM"])[0]
        self.is_mla = False
        self.needs_sequence_state = False
        if self.architecture == "Seturax":
            self._init_seturax(c, dtype, context_length, quantization)
            return
        if self.architecture == "Verozen":
            self._init_verozen(c, dtype, context_length, quantization)
            return
        if self.architecture == "Gatarax":
            self._init_gatarax(c, dtype, context_length, quantization)
            return
        if self.architecture == "Fudonex":
            self._init_fudonex(c, dtype, context_length, quantization)
            return
        self.hidden_size = c["hidden_size"]
        self.num_hidden_layers = c["num_hidden_layers"]
        self.num_attention_heads = c["num_attention_heads"]
        self.num_key_value_heads = c.get("num_key_value_heads", self.num_attention_heads)
        self.head_dim = c.get("head_dim") or self.hidden_size // self.num_attention_heads
        self.v_head_dim = self.head_dim
        self.intermediate_size = c["intermediate_size"]
        self.vocab_size = c["vocab_size"]
        self.rms_norm_eps = c.get("rms_norm_eps", 1e-6)
        self.rope_theta = c.get("rope_theta", 10000.0)
        self.rope_scaling = c.get("rope_scaling")
        self.max_position_embeddings = c.get("max_position_embeddings", 8192)
        self.tie_word_embeddings = c.get("tie_word_embeddings", False)
        self.context_len = context_length or self.max_position_embeddings
        self.quantization = quantization
        want = _DTYPES[dtype] if dtype in _DTYPES else None
        if want is None:
            want = _DTYPES.get(str(c.get("torch_dtype", "bfloat16")), torch.bfloat16)
        self.dtype = want
        self.is_encoder_decoder = False
        # multi-head latent attention (model_config.py:186-204): the cache holds one latent row per token
        arch = self.architecture
        self.is_mla = arch in ("DeepseekV2ForCausalLM", "DeepseekV3ForCausalLM")
        if self.is_mla:
            self.head_dim = 256
            self.kv_lora_rank = c["kv_lora_rank"]
            self.qk_nope_head_dim = c["qk_nope_head_dim"]
            self.qk_rope_head_dim = c["qk_rope_head_dim"]
            self.v_head_dim = c["v_head_dim"]
            self.q_lora_rank = c.get("q_lora_rank")
            self.num_key_value_heads = 1

    def _init_seturax(self, c: dict, dtype: str, context_length: Optional[int], quantization: Optional[str]) -> None:
        """The Seturax design: config.json lists the layers one by one ("layers": [{"type", "mixer": {...}, "mlp":
        {...} | null}]), with the widths under "width" / "vocab", the embedding's constants under "embedding" and the
        norms' epsilon under "norm".  Every layer may have sizes of its own; what the pools and the attention backend
        need as one number is the maximum over the layers."""
        layers = c["layers"]
        for i, spec in enumerate(layers):
            if spec["type"] != "latent_attention":
                raise ValueError(f"Seturax layer {i}: unknown mixer type {spec['type']!r}")
            if spec.get("mlp") is not None and spec["mlp"].get("kind") != "dense":
                raise ValueError(f"Seturax layer {i}: unknown feed-forward kind {spec['mlp'].get('kind')!r}")
        self.layer_specs = layers
        self.hidden_size = c["width"]
        self.vocab_size = c["vocab"]
        self.num_hidden_layers = len(layers)
        self.num_attention_heads = max(s["mixer"]["heads"] for s in layers)
        self.num_key_value_heads = 1
        self.head_dim = max(s["mixer"]["kv_rank"] + s["mixer"]["rot_dim"] for s in layers)
        self.v_head_dim = max(s["mixer"]["kv_rank"] for s in layers)
        self.intermediate_size = max([s["mlp"]["ff"] for s in layers if s.get("mlp")] or [0])
        self.rms_norm_eps = c["norm"]["eps"]
        self.embedding_scale = c["embedding"]["scale"]
        self.bigram = c["embedding"]["bigram"]
        self.logit_scale = c.get("logit_scale", 1.0)
        self.rope_theta = None
        self.rope_scaling = None
        self.tie_word_embeddings = False
        self.max_position_embeddings = context_length or 131072     # the design fixes no longest sequence
        self.context_len = self.max_position_embeddings
        self.quantization = quantization
        self.dtype = _DTYPES.get(dtype) or torch.bfloat16
        self.is_encoder_decoder = False
        self.needs_sequence_state = True     # previous token and previous normed rows travel from step to step
        self.latent_kv = [(s["mixer"]["kv_rank"], s["mixer"]["rot_dim"]) for s in layers]

    def _init_verozen(self, c: dict, dtype: str, context_length: Optional[int], quantization: Optional[str]) -> None:
        """The Verozen design: "layers" lists the layers one by one, {"type": "gla" | "attention" | "retention", "mixer":
        {...}, "mlp": {"kind": "moe", "expert": {"ff"}, "router": {...}} | null}; widths under "width" / "vocab", the
        grouped norm under "norm" {"eps", "groups"}, the residual's weight in front of every norm under "postln_alpha",
        the per-layer token input under "token_side" {"dim"}.  Layers may differ in every size.  Attention layers keep
        keys and values per token (kv_layer_shapes), the two recurrent mixers one matrix per head and sequence
        (recurrent_layer_shapes)."""
        layers = c["layers"]
        for i, spec in enumerate(layers):
            if spec["type"] not in ("gla", "attention", "retention"):
                raise ValueError(f"Verozen layer {i}: unknown mixer type {spec['type']!r}")
            if spec.get("mlp") is not None and spec["mlp"].get("kind", "moe") != "moe":
                raise ValueError(f"Verozen layer {i}: unknown feed-forward kind {spec['mlp'].get('kind')!r}")
            m = spec["mixer"]
            if spec["type"] == "attention":
                if m["heads"] % m.get("kv_heads", m["heads"]):
                    raise ValueError(f"Verozen layer {i}: {m['heads']} query heads over {m['kv_heads']} key heads")
                if m.get("vdim", m["dim"]) != m["dim"]:
                    raise ValueError(f"Verozen layer {i}: the values are the keys, so vdim must equal dim")
            if spec["type"] == "retention" and len(m["decay"]) != m["heads"]:
                raise ValueError(f"Verozen layer {i}: {len(m['decay'])} decays for {m['heads']} heads")
        self.layer_specs = layers
        self.hidden_size = c["width"]
        self.vocab_size = c["vocab"]
        self.num_hidden_layers = len(layers)
        att = [s["mixer"] for s in layers if s["type"] == "attention"]
        self.num_attention_heads = max([m["heads"] for m in att] or [1])
        self.num_key_value_heads = max([m.get("kv_heads", m["heads"]) for m in att] or [1])
        self.head_dim = max([m["dim"] for m in att] or [1])
        self.v_head_dim = self.head_dim
        self.intermediate_size = max([s["mlp"]["expert"]["ff"] for s in layers if s.get("mlp")] or [0])
        self.rms_norm_eps = c["norm"]["eps"]
        self.norm_groups = int(c["norm"].get("groups", 1))
        if self.hidden_size % self.norm_groups:
            raise ValueError(f"Verozen: width {self.hidden_size} is not a multiple of {self.norm_groups} norm groups")
        self.postln_alpha = float(c.get("postln_alpha", 1.0))
        side = c.get("token_side")
        self.token_side_dim = int(side["dim"]) if side else 0
        self.rope_theta = None
        self.rope_scaling = None
        self.tie_word_embeddings = False
        self.max_position_embeddings = context_length or 131072     # the design fixes no longest sequence
        self.context_len = self.max_position_embeddings
        self.quantization = quantization
        self.dtype = _DTYPES.get(dtype) or torch.bfloat16
        self.is_encoder_decoder = False
        self.needs_sequence_state = any(s["type"] != "attention" for s in layers)
        # per layer (kv heads, key width, value width) of the layers that cache keys and values, None for the others
        self.kv_layer_shapes = [(s["mixer"].get("kv_heads", s["mixer"]["heads"]), s["mixer"]["dim"], s["mixer"]["dim"])
                                if s["type"] == "attention" else None for s in layers]
        # per layer (heads, key width, value width) of the state matrices of the recurrent layers, None for the others
        self.recurrent_layer_shapes = [(s["mixer"]["heads"], s["mixer"]["dim"], s["mixer"]["vdim"])
                                       if s["type"] != "attention" else None for s in layers]

    def _init_gatarax(self, c: dict, dtype: str, context_length: Optional[int], quantization: Optional[str]) -> None:
        """The Gatarax design: "layers" lists the layers one by one, {"type": "parallel" | "lightning", "mixer": {...},
        "mlp": {"kind": "dense", "ff"} | {"kind": "moe", "expert": {"ff"}, "router": {...}} | null}; widths under "width" /
        "vocab", the norms' epsilon under "norm", the embedding's factor under "embedding", the taps of the convolution in
        front of every sublayer under "canon", the factor of the logits under "logit_scale".  A "parallel" mixer holds a
        windowed attention branch ("left": keys and values per token, kv_layer_shapes) beside a gated-delta-rule branch
        ("right": one matrix per head and sequence); a "lightning" mixer is a linear recurrence with a fixed decay per
        head.  Layers may differ in every size."""
        layers = c["layers"]
        for i, spec in enumerate(layers):
            if spec["type"] not in ("parallel", "lightning"):
                raise ValueError(f"Gatarax layer {i}: unknown mixer type {spec['type']!r}")
            if spec.get("mlp") is not None and spec["mlp"].get("kind") not in ("dense", "moe"):
                raise ValueError(f"Gatarax layer {i}: unknown feed-forward kind {spec['mlp'].get('kind')!r}")
            m = spec["mixer"]
            if spec["type"] == "parallel":
                for side in ("left", "right"):
                    b = m[side]
                    if b["heads"] % b.get("kv_heads", b["heads"]):
                        raise ValueError(f"Gatarax layer {i} {side}: {b['heads']} heads over {b['kv_heads']} key heads")
            elif len(m["decay"]) != m["heads"]:
                raise ValueError(f"Gatarax layer {i}: {len(m['decay'])} decays for {m['heads']} heads")
        self.layer_specs = layers
        self.hidden_size = c["width"]
        self.vocab_size = c["vocab"]
        self.num_hidden_layers = len(layers)
        att = [s["mixer"]["left"] for s in layers if s["type"] == "parallel"]
        self.num_attention_heads = max([m["heads"] for m in att] or [1])
        self.num_key_value_heads = max([m.get("kv_heads", m["heads"]) for m in att] or [1])
        self.head_dim = max([m["dim"] for m in att] or [1])
        self.v_head_dim = max([m.get("vdim", m["dim"]) for m in att] or [1])
        self.intermediate_size = max([s["mlp"]["ff"] if s["mlp"]["kind"] == "dense" else s["mlp"]["expert"]["ff"]
                                      for s in layers if s.get("mlp")] or [0])
        self.rms_norm_eps = c["norm"]["eps"]
        self.embedding_scale = float((c.get("embedding") or {}).get("scale", 1.0))
        self.canon_taps = int((c.get("canon") or {}).get("taps", 0))
        self.logit_scale = float(c.get("logit_scale", 1.0))
        self.rope_theta = None
        self.rope_scaling = None
        self.tie_word_embeddings = True
        self.max_position_embeddings = context_length or 131072     # the design fixes no longest sequence
        self.context_len = self.max_position_embeddings
        self.quantization = quantization
        self.dtype = _DTYPES.get(dtype) or torch.bfloat16
        self.is_encoder_decoder = False
        self.needs_sequence_state = True      # convolution inputs and recurrent matrices travel from step to step
        self.kv_layer_shapes = [(s["mixer"]["left"].get("kv_heads", s["mixer"]["left"]["heads"]), s["mixer"]["left"]["dim"],
                                 s["mixer"]["left"].get("vdim", s["mixer"]["left"]["dim"]))
                                if s["type"] == "parallel" else None for s in layers]
        self.recurrent_layer_shapes = [(s["mixer"]["right"]["heads"], s["mixer"]["right"]["dim"], s["mixer"]["right"]["vdim"])
                                       if s["type"] == "parallel" else (s["mixer"]["heads"], s["mixer"]["dim"], s["mixer"]["vdim"])
                                       for s in layers]

    def _init_fudonex(self, c: dict, dtype: str, context_length: Optional[int], quantization: Optional[str]) -> None:
        """The Fudonex design: "layers" lists the layers one by one, {"type": "attention" | "mamba2" | "delta", "mixer":
        {...}, "mlp": {"kind": "dense", "ff"} | null}; widths under "width" / "vocab", the norms' epsilon under "norm", the
        embedding's factor under "embedding", the factor on every sublayer's normed output under "residual_mult", the
        cap of the logits under "logit_softcap".  An "attention" mixer keeps keys and values per token (kv_layer_shapes)
        and, with "mask" {"size", "pool"}, averaged blocks of them (kv_layer_pools: the block lengths asked for by the
        layer itself and by the layers that read its cache); with "kv_from": j it keeps none and reads layer j's
        (kv_layer_sources), under a mask of its own.  "mamba2" and "delta" mixers keep one matrix per head and sequence
        (recurrent_layer_shapes).  Layers may differ in every size."""
        layers = c["layers"]
        for i, spec in enumerate(layers):
            if spec["type"] not in ("attention", "mamba2", "delta"):
                raise ValueError(f"Fudonex layer {i}: unknown mixer type {spec['type']!r}")
            if spec.get("mlp") is not None and spec["mlp"].get("kind") != "dense":
                raise ValueError(f"Fudonex layer {i}: unknown feed-forward kind {spec['mlp'].get('kind')!r}")
            m = spec["mixer"]
            if spec["type"] == "attention":
                if m["heads"] % m.get("kv_heads", m["heads"]):
                    raise ValueError(f"Fudonex layer {i}: {m['heads']} query heads over {m['kv_heads']} key heads")
                src = m.get("kv_from")
                if src is not None:
                    if not (0 <= src < i) or layers[src]["type"] != "attention" or layers[src]["mixer"].get("kv_from") is not None:
                        raise ValueError(f"Fudonex layer {i}: kv_from {src} is not an earlier attention layer with keys of its own")
                    s = layers[src]["mixer"]

                    def kv_shape(x):
                        return (x.get("kv_heads", x["heads"]), x["dim"], x.get("vdim", x["dim"]))

                    if kv_shape(s) != kv_shape(m):
                        raise ValueError(f"Fudonex layer {i}: its key / value shapes differ from layer {src}'s")
                rot = m.get("rot")
                if rot and (rot["dims"] % 2 or rot["dims"] > m["dim"]):
                    raise ValueError(f"Fudonex layer {i}: rotation over {rot['dims']} of {m['dim']} features")
            elif spec["type"] == "mamba2":
                if m["heads"] % m.get("groups", 1) or (m["heads"] * m["vdim"]) % m.get("norm_groups", 1):
                    raise ValueError(f"Fudonex layer {i}: heads, groups and norm groups do not divide")
            elif m["heads"] % m.get("kv_heads", m["heads"]):
                raise ValueError(f"Fudonex layer {i}: {m['heads']} heads over {m['kv_heads']} key heads")
        self.layer_specs = layers
        self.hidden_size = c["width"]
        self.vocab_size = c["vocab"]
        self.num_hidden_layers = len(layers)
        att = [s["mixer"] for s in layers if s["type"] == "attention"]
        self.num_attention_heads = max([m["heads"] for m in att] or [1])
        self.num_key_value_heads = max([m.get("kv_heads", m["heads"]) for m in att] or [1])
        self.head_dim = max([m["dim"] for m in att] or [1])
        self.v_head_dim = max([m.get("vdim", m["dim"]) for m in att] or [1])
        self.intermediate_size = max([s["mlp"]["ff"] for s in layers if s.get("mlp")] or [0])
        self.rms_norm_eps = c["norm"]["eps"]
        self.embedding_scale = float((c.get("embedding") or {}).get("scale", 1.0))
        self.residual_mult = float(c.get("residual_mult", 1.0))
        cap = c.get("logit_softcap")
        self.final_logit_softcapping = float(cap) if cap else None
        self.rope_theta = None
        self.rope_scaling = None
        self.tie_word_embeddings = True
        self.max_position_embeddings = context_length or 131072     # the design fixes no longest sequence
        self.context_len = self.max_position_embeddings
        self.quantization = quantization
        self.dtype = _DTYPES.get(dtype) or torch.bfloat16
        self.is_encoder_decoder = False
        self.needs_sequence_state = any(s["type"] != "attention" for s in layers)

        def own_kv(s):
            return s["type"] == "attention" and s["mixer"].get("kv_from") is None

        self.kv_layer_shapes = [(s["mixer"].get("kv_heads", s["mixer"]["heads"]), s["mixer"]["dim"], s["mixer"].get("vdim", s["mixer"]["dim"]))
                                if own_kv(s) else None for s in layers]
        self.kv_layer_sources = {i: int(s["mixer"]["kv_from"]) for i, s in enumerate(layers)
                                 if s["type"] == "attention" and s["mixer"].get("kv_from") is not None}
        # the block lengths of a layer's averaged keys and values: its own mask's and those of the layers that read its cache
        # (a reader has its own mask), so a tuple per owning layer
        pools = []
        for i, s in enumerate(layers):
            sizes = set()
            if own_kv(s):
                readers = [s["mixer"]] + [layers[j]["mixer"] for j, src in self.kv_layer_sources.items() if src == i]
                sizes = {int((r.get("mask") or {}).get("pool", 0) or 0) for r in readers if (r.get("mask") or {}).get("size", 0) > 0}
                sizes.discard(0)
            pools.append(tuple(sorted(sizes)))
        self.kv_layer_pools = pools
        self.recurrent_layer_shapes = [None if s["type"] == "attention" else
                                       (s["mixer"]["heads"], s["mixer"]["state"] if s["type"] == "mamba2" else s["mixer"]["dim"],
                                        s["mixer"]["vdim"]) for s in layers]

    @classmethod
    def from_path(cls, model_path: str, **kw) -> "ModelConfig":
        with open(os.path.join(model_path, "config.json")) as f:
            return cls(json.load(f), **kw)

    def get_num_kv_heads(self, tp_size: int) -> int:
        return max(1, self.num_key_value_heads // tp_size)
