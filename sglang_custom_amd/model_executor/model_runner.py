"""ModelRunner: owns the model, the KV pools, the attention backend and the HIP-graph runner,
and runs one forward pass (python/sglang/srt/model_executor/model_runner.py: ctor :154,
init_memory_pool :1054-1294, init_attention_backend :1305-1391, forward :1535-1600,
forward_decode/extend :1466-1499, sample :1616-1647)."""
import logging
from typing import Dict, Optional, Tuple

import torch

from ..configs.model_config import ModelConfig
from ..distributed import parallel_state
from ..layers.attention.mi355_backend import Mi355AttnBackend
from ..layers.logits_processor import LogitsProcessorOutput
from ..layers.quantization.w8a8_fp8 import W8A8Fp8LinearMethod
from ..layers.sampler import Sampler
from ..mem_cache.allocator import PagedTokenToKVPoolAllocator, TokenToKVPoolAllocator
from ..mem_cache.memory_pool import (
    LatentTokenToKVPool,
    LayeredMHATokenToKVPool,
    MHATokenToKVPool,
    MLATokenToKVPool,
    ReqToTokenPool,
    SequenceStatePool,
)
from ..models.registry import get_model_class
from ..server_args import ServerArgs
from .forward_batch_info import ForwardBatch

logger = logging.getLogger(__name__)


class ModelRunner:
    def __init__(self, model_config: ModelConfig, server_args: ServerArgs, gpu_id: int = 0,
                 tp_rank: int = 0, tp_size: int = 1,
                 weights: Optional[Dict[str, torch.Tensor]] = None, attn_backend_cls=None):
        self.model_config = model_config
        self.server_args = server_args
        self.tp_rank, self.tp_size = tp_rank, tp_size
        self.gpu_id = gpu_id
        self.dtype = model_config.dtype
        if server_args.device == "cuda":
            torch.cuda.set_device(gpu_id)
            self.device = f"cuda:{gpu_id}"
        else:
            self.device = server_args.device
        self.init_torch_distributed()

        quant_factory = None
        if server_args.quantization == "w8a8_fp8":
            quant_factory = W8A8Fp8LinearMethod
        elif server_args.quantization is not None:
            raise ValueError(f"unsupported quantization {server_args.quantization!r}")
        # registry lookup by the configuration's architecture name (model_loader/utils.py of the reference)
        model_cls = get_model_class(getattr(model_config, "architecture", "LlamaForCausalLM"))
        self.model = model_cls(model_config, dtype=self.dtype, device=self.device,
                               quant_method_factory=quant_factory)
        if weights is not None:
            self.model.load_weights(weights)
        else:
            self.model.init_random_weights(seed=server_args.random_seed)
        self.sampler = Sampler()
        # model_runner.py:287-290: the window of sliding-window models (None for Llama / DeepSeek)
        self.sliding_window_size = getattr(self.model, "get_attention_sliding_window_size", lambda: None)()
        self.init_memory_pool()
        self.attn_backend = (attn_backend_cls or Mi355AttnBackend)(self)
        self.graph_runner = None
        self.graph_capture_error = None
        if (not server_args.disable_cuda_graph and str(self.device).startswith("cuda")
                and getattr(self.model, "supports_hip_graph", True)):
            self.init_cuda_graphs()

    def init_cuda_graphs(self):
        """Capture the decode graphs (model_runner.py:1393-1420 of the reference).  The outcome is agreed on
        by all TP ranks: a capture that failed on ONE rank (or a collective of its warm-up runs that gave up
        waiting for that rank) makes every rank take the same road -- raise together, or, with
        server_args.graph_capture_fallback, run eager on this same runner (no second process group, the
        one-launch collectives dropped because a timed-out barrier leaves them unusable)."""
        from .hip_graph_runner import HipGraphRunner

        err = None
        try:
            self.graph_runner = HipGraphRunner(self)
        except Exception as e:  # noqa: BLE001
            err = f"{type(e).__name__}: {e}"
            self.graph_runner = None
        if not parallel_state.tp_any(err is not None):
            return
        self.graph_runner = None
        self.graph_capture_error = err or "graph capture failed on another rank"
        torch.cuda.synchronize()
        if parallel_state.get_custom_all_reduce() is not None:
            parallel_state.drop_custom_all_reduce("dropped after a failed graph capture")
        if not getattr(self.server_args, "graph_capture_fallback", False):
            raise RuntimeError(f"HIP-graph capture failed ({self.graph_capture_error}); "
                               "set disable_cuda_graph or graph_capture_fallback")
        logger.warning("HIP-graph capture failed (%s); running eager", self.graph_capture_error)

    # ---- set-up ----
    def init_torch_distributed(self):
        if self.tp_size == 1:
            parallel_state.init_distributed_environment(1, 0)
            return
        if getattr(self.server_args, "simulate_tp_shard", False):
            parallel_state.init_simulated_shard(self.tp_size, self.tp_rank)
            return
        backend = self.server_args.dist_backend or (
            "nccl" if str(self.device).startswith("cuda") else "gloo")
        parallel_state.init_distributed_environment(
            self.tp_size, self.tp_rank, backend, self.server_args.dist_init_method,
            use_custom_all_reduce=(not self.server_args.disable_custom_all_reduce
                                   and str(self.device).startswith("cuda")),
            local_device=torch.device(self.device).index or 0,
            custom_all_reduce_self_test=self.server_args.custom_all_reduce_self_test)

    def init_memory_pool(self):
        cfg, sa = self.model_config, self.server_args
        kv_heads = cfg.get_num_kv_heads(self.tp_size)
        kvd = getattr(sa, "kv_cache_dtype", "auto") or "auto"
        if kvd not in ("auto", "fp8_e4m3"):
            raise ValueError(f"kv_cache_dtype {kvd!r}: expected 'auto' or 'fp8_e4m3'")
        self.kv_cache_dtype = torch.float8_e4m3fn if kvd == "fp8_e4m3" else self.dtype
        mla = getattr(cfg, "is_mla", False)
        latent = getattr(cfg, "latent_kv", None)     # per-layer (rank, rope width) of a latent cache with unequal layers
        layered = getattr(cfg, "kv_layer_shapes", None)   # per-layer (kv heads, key width, value width) or None per layer
        if layered is not None:
            cell = max(1, sum(h * (dk + dv) for h, dk, dv in filter(None, layered))) * torch.finfo(self.kv_cache_dtype).bits // 8
            # averaged blocks (kv_layer_pools): one more row per block of P slots, or per slot where pages do not hold whole blocks
            page_ = max(1, int(getattr(sa, "page_size", 1) or 1))
            for s, sizes in zip(layered, getattr(cfg, "kv_layer_pools", None) or []):
                for p in (sizes or ()) if s is not None else ():
                    cell += -(-s[0] * (s[1] + s[2]) * (torch.finfo(self.kv_cache_dtype).bits // 8) // (p if page_ % p == 0 else 1))
        elif latent is not None:
            cell = sum(r + d for r, d in latent) * torch.finfo(self.kv_cache_dtype).bits // 8
        elif mla:
            # one latent row per token and layer (model_runner.py:950-957)
            cell = (cfg.kv_lora_rank + cfg.qk_rope_head_dim) * cfg.num_hidden_layers * torch.finfo(self.kv_cache_dtype).bits // 8
        else:
            cell = 2 * kv_heads * cfg.head_dim * cfg.num_hidden_layers * torch.finfo(self.kv_cache_dtype).bits // 8
        if sa.max_total_tokens is not None:
            self.max_total_num_tokens = sa.max_total_tokens
        else:
            # reference rule: rest_memory * fraction / bytes-per-token (model_runner.py:959-970)
            free, _ = torch.cuda.mem_get_info(self.gpu_id)
            self.max_total_num_tokens = int(free * sa.mem_fraction_static) // cell
        max_reqs = sa.max_running_requests or min(
            max(self.max_total_num_tokens // cfg.context_len * 512, 2048), 4096)
        self.req_to_token_pool = ReqToTokenPool(max_reqs, cfg.context_len + 4, self.device)
        if getattr(self.model, "needs_sequence_state", False):
            # one state slot per request that can be live at a time
            self.req_to_token_pool.attach_state_pool(
                SequenceStatePool(max_reqs, device=self.device, **self.model.sequence_state_spec()))
        page = max(1, int(getattr(sa, "page_size", 1) or 1))
        # whole pages only (model_runner.py:1101-1106 rounds the same way)
        self.max_total_num_tokens = self.max_total_num_tokens // page * page
        if layered is not None:
            if self.kv_cache_dtype != self.dtype:
                raise ValueError("a cache with per-layer shapes is stored in the model dtype")
            self.token_to_kv_pool = LayeredMHATokenToKVPool(self.max_total_num_tokens, page, self.kv_cache_dtype, layered, self.device,
                                                            shared=getattr(cfg, "kv_layer_sources", None),
                                                            pooled=getattr(cfg, "kv_layer_pools", None))
        elif latent is not None:
            if self.kv_cache_dtype != self.dtype:
                raise ValueError("a latent cache with per-layer widths is stored in the model dtype")
            self.token_to_kv_pool = LatentTokenToKVPool(self.max_total_num_tokens, page, self.kv_cache_dtype, latent, self.device)
        elif mla:
            # model_runner.py:1192-1206
            self.token_to_kv_pool = MLATokenToKVPool(
                self.max_total_num_tokens, page, self.kv_cache_dtype, cfg.kv_lora_rank, cfg.qk_rope_head_dim,
                cfg.num_hidden_layers, self.device)
        else:
            layout = getattr(sa, "kv_layout", "auto")
            if layout not in ("auto", "token_major", "head_major"):
                raise ValueError(f"kv_layout {layout!r}: expected auto, token_major or head_major")
            head_major = layout == "head_major" or (
                layout == "auto" and str(self.device).startswith("cuda")
                and self.dtype in (torch.bfloat16, torch.float16) and cfg.head_dim % 8 == 0)
            self.token_to_kv_pool = MHATokenToKVPool(
                self.max_total_num_tokens, page, self.kv_cache_dtype, kv_heads, cfg.head_dim,
                cfg.num_hidden_layers, self.device, head_major=head_major)
        if page == 1:
            self.token_to_kv_pool_allocator = TokenToKVPoolAllocator(
                self.max_total_num_tokens, self.dtype, self.device, self.token_to_kv_pool)
        else:
            self.token_to_kv_pool_allocator = PagedTokenToKVPoolAllocator(
                self.max_total_num_tokens, page, self.dtype, self.device, self.token_to_kv_pool)

    # ---- forward ----
    def forward_decode(self, forward_batch: ForwardBatch) -> LogitsProcessorOutput:
        self.attn_backend.init_forward_metadata(forward_batch)
        return self.model.forward(forward_batch.input_ids, forward_batch.positions, forward_batch)

    def forward_extend(self, forward_batch: ForwardBatch) -> LogitsProcessorOutput:
        self.attn_backend.init_forward_metadata(forward_batch)
        return self.model.forward(forward_batch.input_ids, forward_batch.positions, forward_batch)

    def forward(self, forward_batch: ForwardBatch) -> Tuple[LogitsProcessorOutput, bool]:
        """Returns (logits_output, ran_under_graph) like the reference's forward (:1535-1560)."""
        mode = forward_batch.forward_mode
        if mode.is_decode() and self.graph_runner is not None and self.graph_runner.can_run(forward_batch):
            return self.graph_runner.replay(forward_batch), True
        if mode.is_decode():
            return self.forward_decode(forward_batch), False
        if mode.is_extend():
            return self.forward_extend(forward_batch), False
        raise ValueError(f"Invalid forward mode: {mode}")

    def sample(self, logits_output: LogitsProcessorOutput, forward_batch: ForwardBatch) -> torch.Tensor:
        return self.sampler(logits_output, forward_batch.sampling_info, forward_batch.return_logprob)
