"""torch.Tensor front-end of the C ABI (include/mi355_hotpath.h).

Each function checks device / dtype / contiguity (raising like the reference's
CHECK_INPUT / TORCH_CHECK do, sgl-kernel/csrc/torch_extension_rocm.cc), then passes raw
pointers and the current torch stream to libmi355_hotpath.so.  Nothing here computes: PyTorch
is used for memory and streams only.  Outputs are allocated by the caller or returned fresh,
mirroring sgl-kernel/python/sgl_kernel/{elementwise,sampling}.py.
"""
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import BF16, F16, F32, I32, I64, check

_DT = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}
_IT = {torch.int32: I32, torch.int64: I64}


def _lib_():
    return _lib.load()


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype}; expected float32/bfloat16/float16")


def _gpu(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError("mi355 hot-path ops need tensors on the GPU (no CPU fallback)")


KV_FP8 = 0x100   # MI355_KV_FP8: OR'ed into the dtype code when the KV cache holds e4m3fn bytes


KV_HEAD_MAJOR = 0x200   # MI355_KV_HEAD_MAJOR: the [slots, heads, d] cache tensors are views of [heads, slots, d] memory


KV_INTERLEAVED = 0x400  # MI355_KV_INTERLEAVED: ... of [heads, slots, 2, d] memory, keys in [..., 0, :], values in [..., 1, :]


def _kv_layout(buf: torch.Tensor) -> int:
    """0 for a contiguous [slots, heads, d] cache tensor, KV_HEAD_MAJOR for the permute(1, 0, 2) view of a
    contiguous [heads, slots, d] one, KV_HEAD_MAJOR | KV_INTERLEAVED for one half of a contiguous
    [heads, slots, 2, d] one seen the same way; anything else is refused."""
    if buf.is_contiguous():
        return 0
    assert buf.dim() == 3 and buf.stride(2) == 1, f"KV cache tensor with strides {buf.stride()}"
    s, _, d = buf.shape
    if buf.stride() == (d, s * d, 1):
        return KV_HEAD_MAJOR
    assert buf.stride() == (2 * d, 2 * s * d, 1), \
        f"KV cache tensor is neither [slots, heads, d] contiguous nor a head-major view: strides {buf.stride()}"
    return KV_HEAD_MAJOR | KV_INTERLEAVED


def _kvdt(t: torch.Tensor, cache: torch.Tensor, v_cache: Optional[torch.Tensor] = None) -> int:
    """dtype code of the 16-bit tensors, flagged when `cache` is an fp8 KV buffer and when it is head-major."""
    lay = _kv_layout(cache)
    if v_cache is not None:
        assert _kv_layout(v_cache) == lay and v_cache.shape[0] == cache.shape[0], "k and v cache layouts differ"
        if lay & KV_INTERLEAVED:
            assert (v_cache.shape == cache.shape
                    and v_cache.data_ptr() == cache.data_ptr() + cache.shape[2] * cache.element_size()), \
                "an interleaved cache holds a token's value row right behind its key row"
    return _dt(t) | (KV_FP8 if cache.dtype == torch.float8_e4m3fn else 0) | lay


def _p(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


# ---------------------------------------------------------------------------------- norms
def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float,
            out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """sgl_kernel.rmsnorm(input, weight, eps, out) (sgl-kernel/python/sgl_kernel/elementwise.py)."""
    _gpu(x, weight)
    assert x.dim() == 2 and x.stride(1) == 1 and weight.is_contiguous()
    assert weight.dtype == x.dtype and weight.numel() == x.shape[1]
    if out is None:
        out = torch.empty((x.shape[0], x.shape[1]), dtype=x.dtype, device=x.device)
    assert out.stride(1) == 1 and out.shape == x.shape and out.dtype == x.dtype
    if x.numel() == 0:
        return out
    check(_lib_().mi355_rmsnorm(out.data_ptr(), x.data_ptr(), weight.data_ptr(), x.shape[0],
                                x.shape[1], x.stride(0), out.stride(0), float(eps), _dt(x),
                                _stream(x)), "rmsnorm")
    return out


def fused_add_rmsnorm(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,
                      eps: float) -> None:
    """In place on x and residual (sgl_kernel.fused_add_rmsnorm)."""
    _gpu(x, residual, weight)
    assert x.dim() == 2 and x.is_contiguous() and residual.is_contiguous()
    assert residual.shape == x.shape and residual.dtype == x.dtype == weight.dtype
    if x.numel() == 0:
        return
    check(_lib_().mi355_fused_add_rmsnorm(x.data_ptr(), residual.data_ptr(), weight.data_ptr(),
                                          x.shape[0], x.shape[1], float(eps), _dt(x), _stream(x)),
          "fused_add_rmsnorm")


def silu_and_mul(x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """sgl_kernel.silu_and_mul(input, out): out = silu(x[..., :d]) * x[..., d:]."""
    _gpu(x)
    assert x.is_contiguous() and x.shape[-1] % 2 == 0
    d = x.shape[-1] // 2
    rows = x.numel() // (2 * d)
    if out is None:
        out = torch.empty(x.shape[:-1] + (d,), dtype=x.dtype, device=x.device)
    assert out.is_contiguous() and out.dtype == x.dtype
    if x.numel() == 0:
        return out
    check(_lib_().mi355_silu_and_mul(out.data_ptr(), x.data_ptr(), rows, d, _dt(x), _stream(x)),
          "silu_and_mul")
    return out


def softcap_inplace(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """fused_softcap(full_logits, final_logit_softcapping) (logits_processor.py:607-618): in place,
    fp32, logits <- cap * tanh(logits / cap)."""
    _gpu(logits)
    assert logits.dtype == torch.float32 and logits.is_contiguous() and cap > 0
    check(_lib_().mi355_softcap_inplace(logits.data_ptr(), logits.numel(), float(cap), _stream(logits)),
          "softcap_inplace")
    return logits


# ---------------------------------------------------------------------------------- rope / kv
def rope_inplace(positions: torch.Tensor, q: torch.Tensor, k: torch.Tensor, head_size: int,
                 cos_sin_cache: torch.Tensor, is_neox: bool, v: Optional[torch.Tensor] = None,
                 k_buffer: Optional[torch.Tensor] = None, v_buffer: Optional[torch.Tensor] = None,
                 loc: Optional[torch.Tensor] = None) -> None:
    """apply_rope_with_cos_sin_cache_inplace(positions, query, key, head_size, cos_sin_cache,
    is_neox) (sgl-kernel/python/sgl_kernel/elementwise.py), optionally fused with the KV-cache
    write of MHATokenToKVPool.set_kv_buffer when k_buffer/v_buffer/loc/v are given.
    q: [T, Hq*D], k: [T, Hkv*D] (row-strided views allowed, last dim contiguous)."""
    _gpu(positions, q, k, cos_sin_cache)
    assert positions.dtype == torch.int64 and positions.is_contiguous()
    T = positions.numel()
    q2, k2 = q.view(T, -1), k.view(T, -1)
    assert q2.stride(1) == 1 and k2.stride(1) == 1
    hq, hkv = q2.shape[1] // head_size, k2.shape[1] // head_size
    rotary_dim = cos_sin_cache.shape[1]
    assert cos_sin_cache.is_contiguous()
    cache_dt = _dt(cos_sin_cache)
    fused = k_buffer is not None
    if fused:
        assert v is not None and v_buffer is not None and loc is not None
        v2 = v.view(T, -1)
        assert v2.stride(1) == 1
        assert k_buffer.dtype == q.dtype and v_buffer.dtype == q.dtype and v.dtype == q.dtype
        assert loc.is_contiguous() and loc.numel() == T
    check(_lib_().mi355_rope_inplace(
        q2.data_ptr(), k2.data_ptr(), _p(v) if fused else None, positions.data_ptr(),
        cos_sin_cache.data_ptr(), cache_dt, T, hq, hkv, head_size, rotary_dim, q2.stride(0),
        k2.stride(0), v.view(T, -1).stride(0) if fused else 0, 1 if is_neox else 0,
        _p(k_buffer) if fused else None, _p(v_buffer) if fused else None,
        _p(loc) if fused else None, _IT[loc.dtype] if fused else I64,
        k_buffer.shape[0] if fused else 0, _kvdt(q, k_buffer, v_buffer) if fused else _dt(q), _stream(q)), "rope_inplace")


def set_kv_buffer(k_buffer: torch.Tensor, v_buffer: torch.Tensor, loc: torch.Tensor,
                  cache_k: torch.Tensor, cache_v: torch.Tensor) -> None:
    """k_buffer[loc] = cache_k; v_buffer[loc] = cache_v (memory_pool.py:457-458)."""
    _gpu(k_buffer, v_buffer, loc, cache_k, cache_v)
    T = loc.numel()
    k2, v2 = cache_k.view(T, -1), cache_v.view(T, -1)
    assert k2.stride(1) == 1 and v2.stride(1) == 1 and loc.is_contiguous()
    assert cache_k.dtype == cache_v.dtype and k_buffer.dtype == v_buffer.dtype
    assert k_buffer.dtype in (cache_k.dtype, torch.float8_e4m3fn)
    k_row = k_buffer.numel() // k_buffer.shape[0]
    v_row = v_buffer.numel() // v_buffer.shape[0]
    assert k2.shape[1] == k_row and v2.shape[1] == v_row
    kvdt = _kvdt(cache_k, k_buffer, v_buffer)
    if kvdt & KV_HEAD_MAJOR:     # the scatter must know the heads: rows of the cache are not contiguous
        heads = k_buffer.shape[1]
        check(_lib_().mi355_set_kv_buffer_heads(k_buffer.data_ptr(), v_buffer.data_ptr(), k2.data_ptr(), v2.data_ptr(),
                                                loc.data_ptr(), _IT[loc.dtype], T, heads, k_buffer.shape[2],
                                                v_buffer.shape[2], k2.stride(0), v2.stride(0), k_buffer.shape[0],
                                                kvdt, _stream(cache_k)), "set_kv_buffer_heads")
        return
    check(_lib_().mi355_set_kv_buffer(k_buffer.data_ptr(), v_buffer.data_ptr(), k2.data_ptr(),
                                      v2.data_ptr(), loc.data_ptr(), _IT[loc.dtype], T, k_row,
                                      v_row, k2.stride(0), v2.stride(0), k_buffer.shape[0],
                                      kvdt, _stream(cache_k)), "set_kv_buffer")


def embedding(ids: torch.Tensor, table: torch.Tensor, vocab_start: int = 0,
              vocab_end: Optional[int] = None) -> torch.Tensor:
    _gpu(ids, table)
    assert ids.dtype == torch.int64 and ids.is_contiguous() and table.is_contiguous()
    if vocab_end is None:
        vocab_end = vocab_start + table.shape[0]
    out = torch.empty((ids.numel(), table.shape[1]), dtype=table.dtype, device=table.device)
    if ids.numel() == 0:
        return out
    check(_lib_().mi355_embedding(out.data_ptr(), ids.data_ptr(), table.data_ptr(), ids.numel(),
                                  table.shape[1], vocab_start, vocab_end, _dt(table),
                                  _stream(table)), "embedding")
    return out


# ---------------------------------------------------------------------------------- index ops
def create_kv_indices(req_to_token: torch.Tensor, req_pool_indices: torch.Tensor,
                      page_kernel_lens: torch.Tensor, kv_indptr: torch.Tensor,
                      kv_start_idx: Optional[torch.Tensor], kv_indices: torch.Tensor) -> None:
    """create_flashinfer_kv_indices_triton[(bs,)](...) (layers/attention/utils.py:5-41)."""
    _gpu(req_to_token, req_pool_indices, page_kernel_lens, kv_indptr, kv_indices)
    assert req_to_token.dtype == torch.int32 and req_to_token.stride(1) == 1
    assert kv_indptr.dtype == torch.int32 and kv_indices.dtype == torch.int32
    assert kv_start_idx is None or kv_start_idx.dtype == torch.int32
    bs = req_pool_indices.numel()
    check(_lib_().mi355_create_kv_indices(
        req_to_token.data_ptr(), req_pool_indices.data_ptr(), _IT[req_pool_indices.dtype],
        page_kernel_lens.data_ptr(), _IT[page_kernel_lens.dtype], kv_indptr.data_ptr(),
        _p(kv_start_idx), kv_indices.data_ptr(), req_to_token.stride(0), bs,
        _stream(req_to_token)), "create_kv_indices")


def write_req_to_token(req_to_token: torch.Tensor, req_pool_indices: torch.Tensor,
                       pre_lens: torch.Tensor, seq_lens: torch.Tensor, extend_lens: torch.Tensor,
                       out_cache_loc: torch.Tensor) -> None:
    """write_req_to_token_pool_triton[(bs,)](...) (managers/schedule_batch.py:1900-1934)."""
    _gpu(req_to_token, req_pool_indices, pre_lens, seq_lens, extend_lens, out_cache_loc)
    for t in (req_pool_indices, pre_lens, seq_lens, extend_lens, out_cache_loc):
        assert t.dtype == torch.int64 and t.is_contiguous()
    assert req_to_token.dtype == torch.int32 and req_to_token.stride(1) == 1
    check(_lib_().mi355_write_req_to_token(
        req_to_token.data_ptr(), req_pool_indices.data_ptr(), pre_lens.data_ptr(),
        seq_lens.data_ptr(), extend_lens.data_ptr(), out_cache_loc.data_ptr(),
        req_to_token.stride(0), req_pool_indices.numel(), _stream(req_to_token)),
        "write_req_to_token")


def compute_position(extend_prefix_lens: torch.Tensor, extend_seq_lens: torch.Tensor,
                     extend_seq_lens_sum: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """compute_position_triton (model_executor/forward_batch_info.py:703-726)."""
    _gpu(extend_prefix_lens, extend_seq_lens)
    assert extend_prefix_lens.dtype == torch.int32 and extend_seq_lens.dtype == torch.int32
    bs = extend_seq_lens.numel()
    dev = extend_seq_lens.device
    positions = torch.empty(extend_seq_lens_sum, dtype=torch.int64, device=dev)
    extend_start_loc = torch.empty(bs, dtype=torch.int32, device=dev)
    check(_lib_().mi355_compute_position(extend_prefix_lens.data_ptr(), extend_seq_lens.data_ptr(),
                                         positions.data_ptr(), extend_start_loc.data_ptr(), bs,
                                         _stream(extend_seq_lens)), "compute_position")
    return positions, extend_start_loc


def prepare_decode(req_to_token: torch.Tensor, req_pool_indices: torch.Tensor,
                   seq_lens: torch.Tensor, out_cache_loc: torch.Tensor,
                   positions: torch.Tensor) -> None:
    """In place: seq_lens += 1; positions = clamp(seq_lens-1, 0);
    req_to_token[req_pool_indices, seq_lens-1] = out_cache_loc
    (managers/schedule_batch.py:1543-1573, forward_batch_info.py:776-778)."""
    _gpu(req_to_token, req_pool_indices, seq_lens, out_cache_loc, positions)
    for t in (req_pool_indices, seq_lens, out_cache_loc, positions):
        assert t.dtype == torch.int64 and t.is_contiguous()
    check(_lib_().mi355_prepare_decode(req_to_token.data_ptr(), req_pool_indices.data_ptr(),
                                       seq_lens.data_ptr(), out_cache_loc.data_ptr(),
                                       positions.data_ptr(), req_to_token.stride(0),
                                       seq_lens.numel(), _stream(seq_lens)), "prepare_decode")


def copy_decode_inputs(dsts, srcs, n: int) -> None:
    """dsts[i][:n] = srcs[i][:n] for up to five int64 device vectors in one launch (the static inputs
    of a captured decode step, cuda_graph_runner.py:652-676)."""
    import ctypes

    assert 1 <= len(dsts) == len(srcs) <= 5
    for d, s_ in zip(dsts, srcs):
        _gpu(d, s_)
        assert d.dtype == s_.dtype == torch.int64 and d.is_contiguous() and s_.is_contiguous()
        assert d.numel() >= n and s_.numel() >= n
    arr = ctypes.c_void_p * len(dsts)
    check(_lib_().mi355_copy_decode_inputs(arr(*[d.data_ptr() for d in dsts]), arr(*[s_.data_ptr() for s_ in srcs]),
                                           len(dsts), n, _stream(dsts[0])), "copy_decode_inputs")


def alloc_extend_pages(prefix_lens: torch.Tensor, seq_lens: torch.Tensor, last_loc: torch.Tensor,
                       free_pages: torch.Tensor, page_size: int, extend_num_tokens: int):
    """Page-aligned slots for an extend batch (allocator.py:276-360).  Returns (out_indices int64
    [extend_num_tokens], pages consumed from the front of free_pages).  The caller made sure
    free_pages holds enough pages."""
    _gpu(prefix_lens, seq_lens, last_loc, free_pages)
    for t in (prefix_lens, seq_lens, last_loc, free_pages):
        assert t.dtype == torch.int64 and t.is_contiguous()
    bs = seq_lens.numel()
    out = torch.empty(extend_num_tokens, dtype=torch.int64, device=seq_lens.device)
    totals = torch.zeros(2, dtype=torch.int64, device=seq_lens.device)
    check(_lib_().mi355_alloc_extend(prefix_lens.data_ptr(), seq_lens.data_ptr(), last_loc.data_ptr(),
                                     free_pages.data_ptr(), out.data_ptr(), totals.data_ptr(), bs, page_size,
                                     _stream(seq_lens)), "alloc_extend")
    pages, tokens = totals.tolist()
    assert tokens == extend_num_tokens, (tokens, extend_num_tokens)
    return out, pages


def alloc_decode_pages(seq_lens: torch.Tensor, last_loc: torch.Tensor, free_pages: torch.Tensor, page_size: int):
    """One slot per request for a decode step (allocator.py:364-401); seq_lens counts the new token.
    Returns (out_indices int64 [bs], pages consumed)."""
    _gpu(seq_lens, last_loc, free_pages)
    for t in (seq_lens, last_loc, free_pages):
        assert t.dtype == torch.int64 and t.is_contiguous()
    bs = seq_lens.numel()
    out = torch.empty(bs, dtype=torch.int64, device=seq_lens.device)
    totals = torch.zeros(2, dtype=torch.int64, device=seq_lens.device)
    check(_lib_().mi355_alloc_decode(seq_lens.data_ptr(), last_loc.data_ptr(), free_pages.data_ptr(), out.data_ptr(),
                                     totals.data_ptr(), bs, page_size, _stream(seq_lens)), "alloc_decode")
    return out, int(totals[0].item())


# ---------------------------------------------------------------------------------- attention
def _tickets(t, need: int):
    """Device pointer of the split-merge arrival counters (None: the splits are merged by a second launch)."""
    if t is None:
        return None
    if not (t.is_cuda and t.dtype == torch.int32 and t.is_contiguous() and t.numel() >= need):
        raise _lib.Mi355Error(f"split tickets must be >= {need} contiguous int32 counters on the GPU")
    return t.data_ptr()


def _chunk(t):
    """Device pointer of the batch's keys-per-split value (None: every sequence is cut into num_kv_splits)."""
    if t is None:
        return None
    if not (t.is_cuda and t.dtype == torch.int32 and t.numel() >= 1):
        raise _lib.Mi355Error("kv_chunk_keys must be an int32 tensor on the GPU")
    return t.data_ptr()


def _split_scratch(attn_logits, attn_lse, rows: int, dv: int, splits: int) -> None:
    """The kernels write rows * splits partial outputs of dv floats and as many log-sum-exps: refuse a
    scratch pair that cannot hold them (the C ABI sees raw pointers and cannot).  Raises Mi355Error
    before anything is launched; not an assert, so that `python -O` keeps the refusal."""
    if splits <= 1:
        return
    if attn_logits is None or attn_lse is None:
        raise _lib.Mi355Error(f"num_kv_splits = {splits} needs attn_logits / attn_lse scratch")
    if not (attn_logits.is_cuda and attn_lse.is_cuda and attn_logits.dtype == attn_lse.dtype == torch.float32
            and attn_logits.is_contiguous() and attn_lse.is_contiguous()):
        raise _lib.Mi355Error("split scratch must be contiguous float32 tensors on the GPU")
    if attn_logits.numel() < rows * splits * dv or attn_lse.numel() < rows * splits:
        raise _lib.Mi355Error(
            f"split scratch too small for {rows} rows x {splits} splits x {dv}: attn_logits holds "
            f"{attn_logits.numel()} floats (needs {rows * splits * dv}), attn_lse {attn_lse.numel()} (needs {rows * splits})")


def decode_num_splits(bs: int, hkv: int, max_seq_len: int, max_splits: int) -> int:
    return _lib_().mi355_decode_num_splits(bs, hkv, max_seq_len, max_splits)


def decode_attention_fwd(q, k_buffer, v_buffer, o, kv_indptr, kv_indices, attn_logits, attn_lse,
                         num_kv_splits: int, max_kv_splits: int, sm_scale: float,
                         logit_cap: float = 0.0, tickets=None, kv_chunk_keys=None) -> None:
    """decode_attention_fwd(...) of the Triton backend (triton_ops/decode_attention.py:677-728),
    kv_indptr/kv_indices addressing.  num_kv_splits is one int for the whole batch.
    tickets: see decode_attention_paged."""
    _gpu(q, k_buffer, v_buffer, o, kv_indptr, kv_indices)
    B, Hq, D = q.shape
    Hkv, Dv = v_buffer.shape[1], v_buffer.shape[2]
    assert q.stride(2) == 1 and q.stride(1) == D and o.is_contiguous()
    assert kv_indptr.dtype == torch.int32 and kv_indices.dtype == torch.int32
    assert num_kv_splits <= max_kv_splits
    _split_scratch(attn_logits, attn_lse, B * Hq, Dv, num_kv_splits)
    check(_lib_().mi355_decode_attention(
        q.data_ptr(), k_buffer.data_ptr(), v_buffer.data_ptr(), o.data_ptr(),
        kv_indices.data_ptr(), 1, None, None, kv_indptr.data_ptr(), 0, _p(attn_logits),
        _p(attn_lse), _tickets(tickets, B * Hq), _chunk(kv_chunk_keys), num_kv_splits, B, Hq, Hkv, D, Dv, q.stride(0), k_buffer.shape[0], float(sm_scale),
        float(logit_cap), _kvdt(q, k_buffer, v_buffer), _stream(q)), "decode_attention")


def decode_attention_paged(q, k_buffer, v_buffer, o, req_to_token, req_pool_indices, seq_lens,
                           attn_logits, attn_lse, num_kv_splits: int, sm_scale: float,
                           logit_cap: float = 0.0, tickets=None, kv_chunk_keys=None) -> None:
    """decode_attention_cpu-style addressing (sgl-kernel/csrc/cpu/decode.cpp:1375): the kernel
    reads req_to_token[req_pool_indices[b], :seq_lens[b]] directly, no kv_indices gather.
    tickets (optional): >= B * Hq int32 arrival counters, zero between calls (the kernel leaves them
    zero); with them the KV splits are merged inside the attention launch instead of by a second one."""
    _gpu(q, k_buffer, v_buffer, o, req_to_token, req_pool_indices, seq_lens)
    B, Hq, D = q.shape
    Hkv, Dv = v_buffer.shape[1], v_buffer.shape[2]
    assert q.stride(2) == 1 and q.stride(1) == D and o.is_contiguous()
    assert req_to_token.dtype == torch.int32 and req_to_token.stride(1) == 1
    assert req_pool_indices.dtype == torch.int64 and seq_lens.dtype == torch.int64
    _split_scratch(attn_logits, attn_lse, B * Hq, Dv, num_kv_splits)
    check(_lib_().mi355_decode_attention(
        q.data_ptr(), k_buffer.data_ptr(), v_buffer.data_ptr(), o.data_ptr(),
        req_to_token.data_ptr(), 0, req_pool_indices.data_ptr(), seq_lens.data_ptr(), None,
        req_to_token.stride(0), _p(attn_logits), _p(attn_lse), _tickets(tickets, B * Hq), _chunk(kv_chunk_keys), num_kv_splits, B, Hq, Hkv, D, Dv,
        q.stride(0), k_buffer.shape[0], float(sm_scale), float(logit_cap), _kvdt(q, k_buffer, v_buffer), _stream(q)),
        "decode_attention")


def decode_attention_paged_static(q, k_buffer, v_buffer, o, req_to_token, req_pool_indices, seq_lens,
                                  num_kv_splits: int, sm_scale: float, logit_cap: float = 0.0) -> None:
    """decode_attention_paged without caller scratch: the split partials live in the library's own
    fixed device array (mi355_decode_attention_static), so the call allocates nothing.  Calls that
    may overlap on one GPU race on that array."""
    _gpu(q, k_buffer, v_buffer, o, req_to_token, req_pool_indices, seq_lens)
    B, Hq, D = q.shape
    Hkv, Dv = v_buffer.shape[1], v_buffer.shape[2]
    assert q.stride(2) == 1 and q.stride(1) == D and o.is_contiguous()
    assert req_to_token.dtype == torch.int32 and req_to_token.stride(1) == 1
    assert req_pool_indices.dtype == torch.int64 and seq_lens.dtype == torch.int64
    check(_lib_().mi355_decode_attention_static(
        q.data_ptr(), k_buffer.data_ptr(), v_buffer.data_ptr(), o.data_ptr(),
        req_to_token.data_ptr(), 0, req_pool_indices.data_ptr(), seq_lens.data_ptr(), None,
        req_to_token.stride(0), num_kv_splits, B, Hq, Hkv, D, Dv,
        q.stride(0), k_buffer.shape[0], float(sm_scale), float(logit_cap), _kvdt(q, k_buffer, v_buffer), _stream(q)),
        "decode_attention_static")


def decode_attention_fused_qkv(qkv_part, positions, out_cache_loc, cos_sin_cache, k_buffer, v_buffer, o, req_to_token,
                               req_pool_indices, seq_lens, attn_logits, attn_lse, num_kv_splits: int,
                               sm_scale: float, part_x_scale=None, part_w_scale=None, tickets=None, kv_chunk_keys=None) -> None:
    """Decode attention straight from the qkv GEMM's split-K partials [splits, B, (Hq + 2 Hkv) * D]:
    sums them, applies neox RoPE to q and the new k, writes the new k / v rows into cache slot
    out_cache_loc[b] (= req_to_token[req_pool_indices[b], seq_lens[b] - 1] for real rows) and attends.  o: [B, Hq, D]."""
    _gpu(qkv_part, positions, cos_sin_cache, k_buffer, v_buffer, o, req_to_token, req_pool_indices, seq_lens)
    B, Hq, D = o.shape
    Hkv = k_buffer.shape[1]
    assert qkv_part.dim() == 3 and qkv_part.is_contiguous() and qkv_part.dtype == torch.float32
    assert qkv_part.shape[1] == B and qkv_part.shape[2] == (Hq + 2 * Hkv) * D
    assert o.is_contiguous()
    assert k_buffer.shape[1:] == (Hkv, D) and v_buffer.shape == k_buffer.shape
    assert k_buffer.dtype == v_buffer.dtype and k_buffer.dtype in (o.dtype, torch.float8_e4m3fn)
    assert positions.dtype == torch.int64 and positions.is_contiguous() and positions.numel() == B
    assert out_cache_loc.dtype == torch.int64 and out_cache_loc.is_contiguous() and out_cache_loc.numel() == B
    assert cos_sin_cache.is_contiguous() and cos_sin_cache.shape[1] == D
    assert req_to_token.dtype == torch.int32 and req_to_token.stride(1) == 1
    assert req_pool_indices.dtype == torch.int64 and seq_lens.dtype == torch.int64
    if part_x_scale is not None:   # partials of an fp8 GEMM: its per-token / per-channel scales
        assert part_x_scale.dtype == part_w_scale.dtype == torch.float32 and part_x_scale.numel() == B
        assert part_w_scale.numel() == qkv_part.shape[2] and part_x_scale.is_contiguous() and part_w_scale.is_contiguous()
    _split_scratch(attn_logits, attn_lse, B * Hq, D, num_kv_splits)
    check(_lib_().mi355_decode_attention_fused_qkv(
        qkv_part.data_ptr(), qkv_part.shape[0], _p(part_x_scale), _p(part_w_scale), positions.data_ptr(),
        out_cache_loc.data_ptr(), cos_sin_cache.data_ptr(),
        _dt(cos_sin_cache), k_buffer.data_ptr(), v_buffer.data_ptr(), o.data_ptr(), req_to_token.data_ptr(), 0,
        req_pool_indices.data_ptr(), seq_lens.data_ptr(), None, req_to_token.stride(0), _p(attn_logits),
        _p(attn_lse), _tickets(tickets, B * Hq), _chunk(kv_chunk_keys), num_kv_splits, B, Hq, Hkv, D, k_buffer.shape[0], float(sm_scale), _kvdt(o, k_buffer, v_buffer), _stream(o)),
        "decode_attention_fused_qkv")


def decode_attention_mla(q, kv_buffer, o, req_to_token, req_pool_indices, seq_lens, attn_logits,
                         attn_lse, num_kv_splits: int, kv_lora_rank: int, sm_scale: float,
                         logit_cap: float = 0.0, tickets=None, kv_chunk_keys=None) -> None:
    """MQA over the compressed MLA cache (deepseek_v2.py:866-875): kv_buffer [slots, 1, rank + rope],
    q [B, H, rank + rope], o [B, H, rank]; the value is kv_buffer[..., :rank].  kv_buffer may hold
    e4m3fn bytes (kv_cache_dtype fp8_e4m3): the rows are widened exactly on use."""
    _gpu(q, kv_buffer, o, req_to_token, req_pool_indices, seq_lens)
    B, Hq, D = q.shape
    assert kv_buffer.is_contiguous() and kv_buffer.shape[1] == 1 and kv_buffer.shape[2] == D
    assert q.stride(2) == 1 and q.stride(1) == D and o.is_contiguous() and o.shape == (B, Hq, kv_lora_rank)
    assert req_to_token.dtype == torch.int32 and req_to_token.stride(1) == 1
    assert req_pool_indices.dtype == torch.int64 and seq_lens.dtype == torch.int64
    _split_scratch(attn_logits, attn_lse, B * Hq, kv_lora_rank, num_kv_splits)
    check(_lib_().mi355_decode_attention_mla(
        q.data_ptr(), kv_buffer.data_ptr(), o.data_ptr(), req_to_token.data_ptr(), 0,
        req_pool_indices.data_ptr(), seq_lens.data_ptr(), None, req_to_token.stride(0),
        _p(attn_logits), _p(attn_lse), _tickets(tickets, B * Hq), _chunk(kv_chunk_keys), num_kv_splits, B, Hq, kv_lora_rank, D - kv_lora_rank,
        q.stride(0), kv_buffer.shape[0], float(sm_scale), float(logit_cap), _kvdt(q, kv_buffer), _stream(q)),
        "decode_attention_mla")


def decode_attention_mla_fused_rope_supported(kv_lora_rank: int, rope_dim: int, dtype: torch.dtype, cache_dtype: torch.dtype) -> bool:
    return dtype in (torch.bfloat16, torch.float16) and bool(_lib_().mi355_decode_attention_mla_fused_rope_supported(
        kv_lora_rank, rope_dim, _DT[dtype], 1 if cache_dtype == torch.float8_e4m3fn else 0))


def decode_attention_mla_fused_rope(q, k_nope, k_pe, positions, out_cache_loc, cos_sin_cache, is_neox: bool, kv_buffer, o,
                                    req_to_token, req_pool_indices, seq_lens, attn_logits, attn_lse, num_kv_splits: int,
                                    kv_lora_rank: int, sm_scale: float, logit_cap: float = 0.0, tickets=None,
                                    kv_chunk_keys=None) -> None:
    """decode_attention_mla with RoPE and the cache write inside the launch (the reference's ROCm kernel
    decode_attention_fwd_grouped_rope, rocm_mla_decode_rope.py:402-439): q [B, H, rank + rope] with its rope part
    NOT rotated, k_nope [B, rank] (row-strided view allowed), k_pe [B, rope] not rotated (row-strided view allowed);
    rotates both at positions, writes the row [k_nope | rope(k_pe)] to kv_buffer[out_cache_loc] (quantised as
    set_kv_buffer does when the cache is e4m3fn) and attends."""
    _gpu(q, k_nope, k_pe, positions, out_cache_loc, cos_sin_cache, kv_buffer, o, req_to_token, req_pool_indices, seq_lens)
    B, Hq, D = q.shape
    rope = D - kv_lora_rank
    assert kv_buffer.is_contiguous() and kv_buffer.shape[1] == 1 and kv_buffer.shape[2] == D
    assert kv_buffer.dtype in (q.dtype, torch.float8_e4m3fn)
    assert q.stride(2) == 1 and q.stride(1) == D and o.is_contiguous() and o.shape == (B, Hq, kv_lora_rank)
    k_nope2, k_pe2 = k_nope.view(B, -1), k_pe.view(B, -1)
    assert k_nope2.shape[1] == kv_lora_rank and k_pe2.shape[1] == rope and k_nope2.stride(1) == 1 and k_pe2.stride(1) == 1
    assert k_nope2.dtype == q.dtype and k_pe2.dtype == q.dtype
    assert positions.dtype == torch.int64 and positions.is_contiguous() and positions.numel() == B
    assert out_cache_loc.dtype == torch.int64 and out_cache_loc.is_contiguous() and out_cache_loc.numel() == B
    assert cos_sin_cache.is_contiguous() and cos_sin_cache.shape[1] == rope
    assert req_to_token.dtype == torch.int32 and req_to_token.stride(1) == 1
    assert req_pool_indices.dtype == torch.int64 and seq_lens.dtype == torch.int64
    _split_scratch(attn_logits, attn_lse, B * Hq, kv_lora_rank, num_kv_splits)
    check(_lib_().mi355_decode_attention_mla_fused_rope(
        q.data_ptr(), k_nope2.data_ptr(), k_nope2.stride(0), k_pe2.data_ptr(), k_pe2.stride(0), positions.data_ptr(),
        out_cache_loc.data_ptr(), cos_sin_cache.data_ptr(), _dt(cos_sin_cache), 1 if is_neox else 0, kv_buffer.data_ptr(),
        o.data_ptr(), req_to_token.data_ptr(), 0, req_pool_indices.data_ptr(), seq_lens.data_ptr(), None,
        req_to_token.stride(0), _p(attn_logits), _p(attn_lse), _tickets(tickets, B * Hq), _chunk(kv_chunk_keys),
        num_kv_splits, B, Hq, kv_lora_rank, rope, q.stride(0), kv_buffer.shape[0], float(sm_scale), float(logit_cap),
        _kvdt(q, kv_buffer), _stream(q)), "decode_attention_mla_fused_rope")


def mla_latent_norms_supported(q_rank: int, kv_rank: int, rope_dim: int, dtype: torch.dtype) -> bool:
    """Whether mla_latent_norms serves the shape (16-bit; the widths multiples of 8, at most 2048 per part)."""
    return (dtype in (torch.bfloat16, torch.float16) and q_rank % 8 == 0 and kv_rank % 8 == 0 and rope_dim % 8 == 0
            and 0 <= q_rank <= 2048 and 0 < kv_rank and 0 < rope_dim and kv_rank + rope_dim <= 2048)


def mla_latent_norms(q_weight: Optional[torch.Tensor], kv_weight: torch.Tensor, q_rank: int, kv_rank: int, rope_dim: int,
                     eps: float, x: Optional[torch.Tensor] = None, part: Optional[torch.Tensor] = None,
                     part_x_scale: Optional[torch.Tensor] = None, part_w_scale: Optional[torch.Tensor] = None,
                     quant_q_fp8: bool = False):
    """q_a_layernorm and kv_a_layernorm over the two parts of fused_qkv_a_proj_with_mqa's output row
    [q_a | c_kv | k_pe] in one launch (deepseek_v2.py:1193-1232): from x [M, width] (row-strided view allowed) or
    from that GEMM's split-K partials [splits, M, width] (with the fp8 GEMM's scales when it was one).  Returns
    (q_a normed [M, q_rank] or None when q_rank == 0, c_kv normed [M, kv_rank], k_pe [M, rope_dim]), all dense;
    with quant_q_fp8 additionally (e4m3fn [M, q_rank], scale [M, 1]) = per_token_quant_fp8 of the normed q_a."""
    src = part if part is not None else x
    _gpu(src, q_weight, kv_weight)
    dt = kv_weight.dtype
    width = q_rank + kv_rank + rope_dim
    if part is not None:
        assert part.dim() == 3 and part.is_contiguous() and part.dtype == torch.float32 and part.shape[2] == width
        rows = part.shape[1]
    else:
        assert x.dim() == 2 and x.shape[1] == width and x.stride(1) == 1 and x.dtype == dt
        rows = x.shape[0]
    assert kv_weight.is_contiguous() and kv_weight.numel() == kv_rank
    assert (q_weight is None) == (q_rank == 0)
    q_out = None
    if q_rank:
        assert q_weight.is_contiguous() and q_weight.numel() == q_rank and q_weight.dtype == dt
        q_out = torch.empty((rows, q_rank), dtype=dt, device=kv_weight.device)
    kv_out = torch.empty((rows, kv_rank), dtype=dt, device=kv_weight.device)
    pe_out = torch.empty((rows, rope_dim), dtype=dt, device=kv_weight.device)
    q8 = s8 = None
    if quant_q_fp8:
        assert q_rank > 0
        q8 = torch.empty((rows, q_rank), dtype=torch.float8_e4m3fn, device=kv_weight.device)
        s8 = torch.empty((rows, 1), dtype=torch.float32, device=kv_weight.device)
    if rows:
        check(_lib_().mi355_mla_latent_norms(
            _p(q_out), kv_out.data_ptr(), pe_out.data_ptr(), _p(x), x.stride(0) if x is not None else 0, _p(part),
            part.shape[0] if part is not None else 0, _p(part_x_scale), _p(part_w_scale), _p(q_weight),
            kv_weight.data_ptr(), _p(q8), _p(s8), rows, q_rank, kv_rank, rope_dim, float(eps), _dt(kv_weight),
            _stream(kv_weight)), "mla_latent_norms")
    if quant_q_fp8:
        return q_out, kv_out, pe_out, q8, s8
    return q_out, kv_out, pe_out


def mla_absorb_supported(m: int, n: int, k: int, tail: int, dtype: torch.dtype) -> bool:
    """Whether mla_absorb serves the shape (decode-sized batch, 16-bit, MFMA-tileable)."""
    return (dtype in (torch.bfloat16, torch.float16) and 0 <= m <= 64 and n >= 16 and n % 16 == 0 and k >= 32
            and k % 32 == 0 and tail % 8 == 0)


def mla_absorb(a: torch.Tensor, w_t: torch.Tensor, tail: int = 0) -> torch.Tensor:
    """The absorbed products of MLA decode as one launch each (deepseek_v2.py:1234-1262, 1296-1333):
    a [M, H, k + tail] (row- and head-strided view allowed, features contiguous), w_t [H, n, k] (each head's
    matrix with the reduction dimension contiguous) -> out [M, H, n + tail] with out[..., :n] = a[..., :k] @ w_t[h].T
    per head and out[..., n:] = a[..., k:].  M <= 64."""
    _gpu(a, w_t)
    m, heads, feat = a.shape
    hw, n, k = w_t.shape
    assert hw == heads and feat == k + tail and a.stride(2) == 1 and w_t.is_contiguous() and a.dtype == w_t.dtype
    out = torch.empty((m, heads, n + tail), dtype=a.dtype, device=a.device)
    if m:
        check(_lib_().mi355_mla_absorb(out.data_ptr(), a.data_ptr(), w_t.data_ptr(), m, heads, n, k, tail, a.stride(0),
                                       a.stride(1), out.stride(0), out.stride(1), _dt(a), _stream(a)), "mla_absorb")
    return out


def mla_prefill_assemble_supported(nope: int, rope: int, vd: int, rank: int, dtype: torch.dtype) -> bool:
    """Whether mla_prefill_assemble serves the shape (16-bit; widths multiples of 8, rope <= 256)."""
    return (dtype in (torch.bfloat16, torch.float16) and nope % 8 == 0 and rope % 8 == 0 and 0 < rope <= 256
            and vd % 8 == 0 and rank % 8 == 0)


def mla_prefill_assemble(q, kv, k_pe, c_kv, positions, cos_sin_cache, is_neox: bool, kv_cache, out_cache_loc,
                         nope: int, rope: int, vd: int):
    """The glue of MLA's multi-head prefill (deepseek_v2.py:1131-1179) in one launch: q [T, H, nope + rope] gets its
    rope part rotated in place; returns k [T, H, nope + rope] = [kv nope part | rope(k_pe)] and v [T, H, vd] from
    kv [T, H, nope + vd]; writes the latent row [c_kv | rope(k_pe)] to kv_cache[out_cache_loc] (quantised when the
    cache is e4m3fn).  k_pe [T, rope] and c_kv [T, rank] may be row-strided views."""
    _gpu(q, kv, k_pe, c_kv, positions, cos_sin_cache, kv_cache, out_cache_loc)
    T, H, D = q.shape
    rank = c_kv.shape[1]
    assert D == nope + rope and q.stride(2) == 1 and q.stride(1) == D
    assert kv.is_contiguous() and kv.shape == (T, H, nope + vd) and kv.dtype == q.dtype
    assert k_pe.shape == (T, rope) and k_pe.stride(1) == 1 and c_kv.shape[0] == T and c_kv.stride(1) == 1
    assert k_pe.dtype == q.dtype and c_kv.dtype == q.dtype
    assert positions.dtype == torch.int64 and positions.is_contiguous() and positions.numel() == T
    assert out_cache_loc.dtype == torch.int64 and out_cache_loc.is_contiguous() and out_cache_loc.numel() == T
    assert cos_sin_cache.is_contiguous() and cos_sin_cache.shape[1] == rope
    assert kv_cache.is_contiguous() and kv_cache.shape[1] == 1 and kv_cache.shape[2] == rank + rope
    assert kv_cache.dtype in (q.dtype, torch.float8_e4m3fn)
    k = torch.empty((T, H, D), dtype=q.dtype, device=q.device)
    v = torch.empty((T, H, vd), dtype=q.dtype, device=q.device)
    if T:
        check(_lib_().mi355_mla_prefill_assemble(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), kv.data_ptr(), k_pe.data_ptr(), k_pe.stride(0), c_kv.data_ptr(),
            c_kv.stride(0), positions.data_ptr(), cos_sin_cache.data_ptr(), _dt(cos_sin_cache), 1 if is_neox else 0,
            kv_cache.data_ptr(), out_cache_loc.data_ptr(), T, H, nope, rope, vd, rank, q.stride(0), kv_cache.shape[0],
            _kvdt(q, kv_cache), _stream(q)), "mla_prefill_assemble")
    return k, v


def extend_attention_mla_supported(hq: int, kv_lora_rank: int, rope_dim: int, dtype: torch.dtype) -> bool:
    """Whether extend_attention_mla serves the shape (latent row of 512 + 64 features, 16-bit)."""
    return dtype in (torch.bfloat16, torch.float16) and bool(
        _lib_().mi355_extend_attention_mla_supported(hq, kv_lora_rank, rope_dim, _DT[dtype]))


def extend_attention_mla(q, kv_buffer, o, req_to_token, req_pool_indices, seq_lens, qo_indptr,
                         max_extend_len: int, kv_lora_rank: int, sm_scale: float, logit_cap: float = 0.0) -> None:
    """attn_mqa (deepseek_v2.py:866-875) of an extend batch in the absorbed form: request b's new tokens
    (rows qo_indptr[b] .. qo_indptr[b + 1] of q [T, H, rank + rope] and o [T, H, rank]) attend to the
    request's first seq_lens[b] cache rows causally; the new tokens' latent rows are in kv_buffer
    [slots, 1, rank + rope] already.  Four consecutive tokens share one pass over the rows."""
    _gpu(q, kv_buffer, o, req_to_token, req_pool_indices, seq_lens, qo_indptr)
    T, Hq, D = q.shape
    B = req_pool_indices.numel()
    assert kv_buffer.is_contiguous() and kv_buffer.shape[1] == 1 and kv_buffer.shape[2] == D
    assert q.stride(2) == 1 and q.stride(1) == D and o.is_contiguous() and o.shape == (T, Hq, kv_lora_rank)
    assert req_to_token.dtype == torch.int32 and req_to_token.stride(1) == 1
    assert req_pool_indices.dtype == torch.int64 and seq_lens.dtype == torch.int64 and seq_lens.numel() == B
    assert qo_indptr.dtype == torch.int32 and qo_indptr.is_contiguous() and qo_indptr.numel() == B + 1
    check(_lib_().mi355_extend_attention_mla(
        q.data_ptr(), kv_buffer.data_ptr(), o.data_ptr(), req_to_token.data_ptr(), req_pool_indices.data_ptr(),
        seq_lens.data_ptr(), qo_indptr.data_ptr(), req_to_token.stride(0), B, int(max_extend_len), Hq, kv_lora_rank,
        D - kv_lora_rank, q.stride(0), kv_buffer.shape[0], float(sm_scale), float(logit_cap), _dt(q), _stream(q)),
        "extend_attention_mla")


def extend_attention_fwd(q_extend, k_extend, v_extend, o_extend, k_buffer, v_buffer, qo_indptr,
                         kv_indptr, kv_indices, custom_mask, is_causal, mask_indptr,
                         max_len_extend, sm_scale=None, logit_cap=0.0,
                         skip_prefix_custom_mask=True, sliding_window_size=-1) -> None:
    """extend_attention_fwd(...) (triton_ops/extend_attention.py:306-438), same argument order."""
    _gpu(q_extend, k_extend, v_extend, o_extend, k_buffer, v_buffer, qo_indptr, kv_indptr, kv_indices)
    T, Hq, D = q_extend.shape
    Hkv, Dv = v_extend.shape[1], v_extend.shape[2]
    assert q_extend.stride(2) == 1 and q_extend.stride(1) == D
    assert k_extend.stride(2) == 1 and k_extend.stride(1) == D
    assert v_extend.stride(2) == 1 and v_extend.stride(1) == Dv
    assert o_extend.is_contiguous()
    assert qo_indptr.dtype == torch.int32 and kv_indptr.dtype == torch.int32 and kv_indices.dtype == torch.int32
    if sm_scale is None:
        sm_scale = 1.0 / (D ** 0.5)
    if custom_mask is not None:
        assert mask_indptr is not None and mask_indptr.dtype == torch.int64
        if custom_mask.dtype == torch.bool:
            custom_mask = custom_mask.view(torch.uint8)
        assert custom_mask.dtype == torch.uint8
    bs = qo_indptr.numel() - 1
    check(_lib_().mi355_extend_attention(
        q_extend.data_ptr(), k_extend.data_ptr(), v_extend.data_ptr(), o_extend.data_ptr(),
        k_buffer.data_ptr(), v_buffer.data_ptr(), qo_indptr.data_ptr(), kv_indptr.data_ptr(),
        kv_indices.data_ptr(), _p(custom_mask), _p(mask_indptr) if custom_mask is not None else None,
        1 if is_causal else 0, 1 if skip_prefix_custom_mask else 0, bs, int(max_len_extend), Hq,
        Hkv, D, Dv, q_extend.stride(0), k_extend.stride(0), v_extend.stride(0),
        k_buffer.shape[0], float(sm_scale), float(logit_cap), int(sliding_window_size),
        _kvdt(q_extend, k_buffer, v_buffer), _stream(q_extend)), "extend_attention")


# ---------------------------------------------------------------------------------- linear
_WS = {}
_WS_RETIRED = []


def _workspace(device, nbytes: int, tag: str = "linear") -> torch.Tensor:
    """Per-device, per-kernel-family grow-only scratch for split-K partials (allocated outside
    graph capture by the first eager call of each shape; ModelRunner warms every shape up before
    capturing).  Zero-filled at allocation: the 16-bit GEMM keeps its arrival counters at the head
    of the buffer and hands them back zeroed after every launch.  Launches that share a buffer
    must be ordered on one stream."""
    ws = _WS.get((device, tag))
    if ws is None or ws.numel() < nbytes:
        if ws is not None:
            # a captured HIP graph may still hold the old pointer: outgrown buffers stay alive
            _WS_RETIRED.append(ws)
        ws = torch.zeros(max(nbytes, 8 << 20), dtype=torch.uint8, device=device)
        _WS[(device, tag)] = ws
    return ws


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """F.linear(x, weight, bias) (layers/quantization/unquant.py:110-122) through the C ABI:
    weight-streaming MFMA kernel for M <= 64 (bf16/f16), exact tiled kernel otherwise."""
    _gpu(x, weight, bias)
    assert x.dim() == 2 and x.stride(1) == 1 and weight.is_contiguous() and weight.dtype == x.dtype
    M, K = x.shape
    N = weight.shape[0]
    assert weight.shape[1] == K
    out_dtype = out_dtype or x.dtype
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    if M == 0:
        return y
    lib = _lib_()
    need = lib.mi355_linear_workspace_bytes(M, N, K)
    ws = _workspace(x.device, need) if need > 0 else None
    check(lib.mi355_linear(y.data_ptr(), x.data_ptr(), weight.data_ptr(), _p(bias), M, N, K,
                           x.stride(0), _p(ws), ws.numel() if ws is not None else 0, _dt(x),
                           _DT[out_dtype], _stream(x)), "linear")
    return y


def linear_tiled_supported(m: int, n: int, k: int, dtype: torch.dtype, silu_mul: bool = False) -> bool:
    """Whether linear_tiled serves the shape (16-bit, K % 64 == 0, K >= 128, N % 16 == 0)."""
    return dtype in (torch.bfloat16, torch.float16) and bool(
        _lib_().mi355_linear_tiled_supported(m, n, k, _DT[dtype], 1 if silu_mul else 0))


def linear_tiled(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                 silu_mul: bool = False) -> torch.Tensor:
    """Prefill-sized F.linear(x, weight, bias) (layers/quantization/unquant.py:110-122) on the
    256 x 256-tile matrix-core kernel; silu_mul=True applies SiluAndMul (layers/activation.py:55-65)
    to the [gate; up] output in the epilogue and returns [M, N / 2]."""
    _gpu(x, weight, bias)
    assert x.dim() == 2 and x.stride(1) == 1 and weight.is_contiguous() and weight.dtype == x.dtype
    M, K = x.shape
    N = weight.shape[0]
    assert weight.shape[1] == K
    y = torch.empty((M, N // 2 if silu_mul else N), dtype=x.dtype, device=x.device)
    if M == 0:
        return y
    check(_lib_().mi355_linear_tiled(y.data_ptr(), x.data_ptr(), weight.data_ptr(), _p(bias), M, N, K,
                                     x.stride(0), _dt(x), 1 if silu_mul else 0, _stream(x)), "linear_tiled")
    return y


def qkv_proj_rope_tiled_supported(m: int, k: int, hq: int, hkv: int, head_dim: int, rotary_dim: int,
                                  is_neox: bool, dtype: torch.dtype, fp8: bool = False) -> bool:
    """Whether qkv_proj_rope_tiled serves the layer (head_dim = rotary_dim = 128, neox, 16-bit)."""
    return dtype in (torch.bfloat16, torch.float16) and bool(_lib_().mi355_qkv_proj_rope_tiled_supported(
        m, k, hq, hkv, head_dim, rotary_dim, 1 if is_neox else 0, _DT[dtype], 1 if fp8 else 0))


def qkv_proj_rope_tiled(x: torch.Tensor, weight: torch.Tensor, hq: int, hkv: int, head_dim: int,
                        positions: torch.Tensor, cos_sin_cache: torch.Tensor, is_neox: bool,
                        k_buffer: torch.Tensor, v_buffer: torch.Tensor, loc: torch.Tensor,
                        x_scale: Optional[torch.Tensor] = None, w_scale: Optional[torch.Tensor] = None,
                        out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """qkv_proj -> rotary_emb -> set_kv_buffer of a prefill batch (models/llama.py:187-199) as one
    kernel: the 256 x 256-tile projection with neox RoPE and the cache write in its epilogue.
    Returns qkv [M, (hq + 2 hkv) * head_dim] holding rotated q, rotated k and v.  With x_scale / w_scale
    x and weight are e4m3fn (per-token / per-channel scales) and out_dtype names the result dtype."""
    _gpu(x, weight, positions, cos_sin_cache, k_buffer, v_buffer, loc)
    fp8 = x_scale is not None
    dtype = out_dtype if fp8 else x.dtype
    assert x.dim() == 2 and x.stride(1) == 1 and weight.is_contiguous() and weight.dtype == x.dtype
    M, K = x.shape
    N = (hq + 2 * hkv) * head_dim
    assert weight.shape == (N, K)
    assert positions.dtype == torch.int64 and positions.is_contiguous() and positions.numel() == M
    assert cos_sin_cache.is_contiguous() and cos_sin_cache.dim() == 2
    assert k_buffer.dtype == dtype and v_buffer.dtype == dtype
    assert k_buffer[0].numel() == hkv * head_dim and v_buffer[0].numel() == hkv * head_dim
    assert _kv_layout(k_buffer) == _kv_layout(v_buffer) and k_buffer.shape == v_buffer.shape
    assert loc.is_contiguous() and loc.numel() == M
    if fp8:
        assert x.dtype == torch.float8_e4m3fn and x.is_contiguous()
        assert x_scale.dtype == torch.float32 and x_scale.is_contiguous() and x_scale.numel() == M
        assert w_scale.dtype == torch.float32 and w_scale.is_contiguous() and w_scale.numel() == N
    qkv = torch.empty((M, N), dtype=dtype, device=x.device)
    if M == 0:
        return qkv
    check(_lib_().mi355_qkv_proj_rope_tiled(
        qkv.data_ptr(), x.data_ptr(), weight.data_ptr(), _p(x_scale), _p(w_scale), M, K, x.stride(0), hq, hkv,
        head_dim, positions.data_ptr(), cos_sin_cache.data_ptr(), _dt(cos_sin_cache), cos_sin_cache.shape[1],
        1 if is_neox else 0, k_buffer.data_ptr(), v_buffer.data_ptr(), loc.data_ptr(), _IT[loc.dtype],
        k_buffer.shape[0], _DT[dtype] | (_kvdt(qkv, k_buffer, v_buffer) & (KV_HEAD_MAJOR | KV_INTERLEAVED)), _stream(x)),
        "qkv_proj_rope_tiled")
    return qkv


def pack_weight(weight: torch.Tensor) -> torch.Tensor:
    """[N, K] 16-bit weight -> MFMA-fragment-ordered copy for linear_packed (decode GEMMs)."""
    _gpu(weight)
    assert weight.dim() == 2 and weight.is_contiguous() and weight.dtype in (torch.bfloat16, torch.float16)
    N, K = weight.shape
    lib = _lib_()
    out = torch.empty(lib.mi355_packed_weight_elems(N, K), dtype=weight.dtype, device=weight.device)
    check(lib.mi355_pack_weight(out.data_ptr(), weight.data_ptr(), N, K, _dt(weight), _stream(weight)),
          "pack_weight")
    return out


def linear_packed(x: torch.Tensor, weight_packed: torch.Tensor, n: int, bias: Optional[torch.Tensor] = None,
                  out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """linear() for M <= 64 on a weight produced by pack_weight (n = number of output features)."""
    _gpu(x, weight_packed, bias)
    assert x.dim() == 2 and x.stride(1) == 1 and weight_packed.dtype == x.dtype
    M, K = x.shape
    out_dtype = out_dtype or x.dtype
    y = torch.empty((M, n), dtype=out_dtype, device=x.device)
    if M == 0:
        return y
    lib = _lib_()
    assert weight_packed.numel() == lib.mi355_packed_weight_elems(n, K)
    need = lib.mi355_linear_workspace_bytes(M, n, K)
    ws = _workspace(x.device, need) if need > 0 else None
    check(lib.mi355_linear_packed(y.data_ptr(), x.data_ptr(), weight_packed.data_ptr(), _p(bias), M, n, K,
                                  x.stride(0), _p(ws), ws.numel() if ws is not None else 0, _dt(x),
                                  _DT[out_dtype], _stream(x)), "linear_packed")
    return y


def linear_packed_partials(x: torch.Tensor, weight_packed: torch.Tensor, n: int) -> Optional[torch.Tensor]:
    """x @ W^T left as fp32 split-K partials [splits, M, N] for fused_add_rmsnorm_partials to sum
    (None when the shape is not served: the caller then runs linear_packed)."""
    _gpu(x, weight_packed)
    assert x.dim() == 2 and x.stride(1) == 1
    m, k = x.shape
    splits = _lib_().mi355_linear_packed_splits(max(m, 1), n, k)
    if splits <= 0 or m > 64 or x.dtype not in (torch.bfloat16, torch.float16):
        return None
    part = torch.empty((splits, m, n), dtype=torch.float32, device=x.device)
    if m:
        check(_lib_().mi355_linear_packed_partials(part.data_ptr(), x.data_ptr(), weight_packed.data_ptr(), m, n, k,
                                                   x.stride(0), _dt(x), _stream(x)), "linear_packed_partials")
    return part


def fused_add_rmsnorm_partials(part: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,
                               eps: float) -> torch.Tensor:
    """y = sum of the split-K partials (rounded once to residual.dtype), then fused_add_rmsnorm(y,
    residual): returns the normalised rows, residual updated in place."""
    _gpu(part, residual, weight)
    assert part.dim() == 3 and part.is_contiguous() and part.dtype == torch.float32
    assert residual.is_contiguous() and residual.shape == part.shape[1:] and residual.dtype == weight.dtype
    x = torch.empty_like(residual)
    if residual.numel():
        check(_lib_().mi355_fused_add_rmsnorm_partials(x.data_ptr(), residual.data_ptr(), weight.data_ptr(),
                                                       part.data_ptr(), part.shape[0], part.shape[1], part.shape[2],
                                                       float(eps), _dt(residual), _stream(residual)),
              "fused_add_rmsnorm_partials")
    return x


def fp8_packed_partials(xq: torch.Tensor, wq_packed: torch.Tensor, n: int) -> Optional[torch.Tensor]:
    """fp8 x fp8 GEMM of fp8_scaled_mm_packed left as raw fp32 split-K partials [splits, M, N]; the
    consumer applies (sum * x_scale[m]) * w_scale[n].  None when the shape is not served."""
    _gpu(xq, wq_packed)
    assert xq.dim() == 2 and xq.is_contiguous() and xq.dtype == torch.float8_e4m3fn
    m, k = xq.shape
    splits = _lib_().mi355_fp8_packed_splits(max(m, 1), n, k)
    if splits <= 0 or m > 64:
        return None
    part = torch.empty((splits, m, n), dtype=torch.float32, device=xq.device)
    if m:
        check(_lib_().mi355_fp8_packed_partials(part.data_ptr(), xq.data_ptr(), wq_packed.data_ptr(), m, n, k,
                                                _stream(xq)), "fp8_packed_partials")
    return part


def rmsnorm_ex(weight: torch.Tensor, eps: float, x: Optional[torch.Tensor] = None,
               residual: Optional[torch.Tensor] = None, part: Optional[torch.Tensor] = None,
               part_x_scale: Optional[torch.Tensor] = None, part_w_scale: Optional[torch.Tensor] = None,
               quant_fp8: bool = False):
    """General decode row norm: input x or split-K partials [splits, M, hidden] (with the fp8 GEMM's
    scales when they come from one), optional fused add of residual (updated in place), and optionally
    the per-token fp8 quantisation of the result.  Returns (out, xq or None, x_scale or None)."""
    src = part if part is not None else x
    _gpu(src, weight, residual)
    rows, hidden = (part.shape[1], part.shape[2]) if part is not None else x.shape
    dt = weight.dtype
    out = torch.empty((rows, hidden), dtype=dt, device=weight.device)
    if part is not None:
        assert part.is_contiguous() and part.dtype == torch.float32
    else:
        assert x.is_contiguous() and x.dtype == dt
    if residual is not None:
        assert residual.is_contiguous() and residual.shape == (rows, hidden) and residual.dtype == dt
    xq = xs = None
    if quant_fp8:
        xq = torch.empty((rows, hidden), dtype=torch.float8_e4m3fn, device=weight.device)
        xs = torch.empty((rows, 1), dtype=torch.float32, device=weight.device)
    if rows:
        check(_lib_().mi355_rmsnorm_ex(out.data_ptr(), _p(x), _p(residual), weight.data_ptr(), _p(part),
                                       part.shape[0] if part is not None else 0, _p(part_x_scale), _p(part_w_scale),
                                       _p(xq), _p(xs), rows, hidden, float(eps), _dt(weight), _stream(weight)),
              "rmsnorm_ex")
    return out, xq, xs


def silu_and_mul_quant_fp8(x: torch.Tensor, pad_to: Optional[int] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """per_token_quant_fp8(silu_and_mul(x)) in one launch: x [M, 2d] 16-bit -> (e4m3fn [M, d], scale [M, 1]);
    pad_to > d: rows of pad_to bytes with zeros behind the d values (see per_token_quant_fp8)."""
    _gpu(x)
    assert x.dim() == 2 and x.is_contiguous() and x.shape[1] % 2 == 0
    m, d = x.shape[0], x.shape[1] // 2
    qs = max(d, pad_to or 0)
    xq = torch.empty((m, qs), dtype=torch.float8_e4m3fn, device=x.device)
    xs = torch.empty((m, 1), dtype=torch.float32, device=x.device)
    if m:
        check(_lib_().mi355_silu_and_mul_quant_fp8(xq.data_ptr(), xs.data_ptr(), x.data_ptr(), m, d, qs, _dt(x),
                                                   _stream(x)), "silu_and_mul_quant_fp8")
    return xq, xs


def prefetch_next(weight_packed: torch.Tensor, m: int, n: int, k: int, budget_bytes: int = 24 << 20) -> None:
    """Hint: the next rmsnorm / fused_add_rmsnorm launch of this thread also pulls the head of this
    packed weight into L2, in the order the M-row skinny GEMM over it will ask for it (24 MiB of the
    32 MiB of L2 by default).  Results never change; shapes the hint does not serve are ignored."""
    check(_lib_().mi355_prefetch_next(weight_packed.data_ptr(), m, n, k, weight_packed.element_size(),
                                      budget_bytes), "prefetch_next")


def pack_weight_gate_up(weight: torch.Tensor) -> torch.Tensor:
    """[2d, K] = [gate rows | up rows] -> packed copy for linear_packed_silu_mul: every 16-row MFMA
    tile holds 8 gate rows followed by the 8 up rows of the same output features."""
    n2, K = weight.shape
    d = n2 // 2
    assert n2 % 16 == 0
    inter = torch.stack([weight[:d].view(d // 8, 8, K), weight[d:].view(d // 8, 8, K)], dim=1)
    return pack_weight(inter.reshape(n2, K).contiguous())


def linear_packed_silu_mul(x: torch.Tensor, weight_packed: torch.Tensor, n: int) -> torch.Tensor:
    """SiluAndMul(x @ W_gate_up^T) in one kernel (models/llama.py:94-98) for M <= 64 rows;
    weight_packed from pack_weight_gate_up, n = 2d rows, returns [M, d]."""
    _gpu(x, weight_packed)
    assert x.dim() == 2 and x.stride(1) == 1 and weight_packed.dtype == x.dtype
    M, K = x.shape
    y = torch.empty((M, n // 2), dtype=x.dtype, device=x.device)
    if M == 0:
        return y
    lib = _lib_()
    assert weight_packed.numel() == lib.mi355_packed_weight_elems(n, K)
    need = lib.mi355_linear_workspace_bytes(M, n, K)
    ws = _workspace(x.device, need) if need > 0 else None
    check(lib.mi355_linear_packed_silu_mul(y.data_ptr(), x.data_ptr(), weight_packed.data_ptr(), M, n, K,
                                           x.stride(0), _p(ws), ws.numel() if ws is not None else 0,
                                           _dt(x), _stream(x)), "linear_packed_silu_mul")
    return y


def per_token_quant_fp8(x: torch.Tensor, pad_to: Optional[int] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """per_token_group_quant_fp8(x, group_size=K) (fp8_kernel.py:115-155) -> (xq e4m3fn, scale [M,1]).
    pad_to > K: xq is [M, pad_to] with zeros behind the K values of every row -- the activation of a packed GEMM
    whose reduction length was rounded up with zero weights."""
    _gpu(x)
    assert x.dim() == 2 and x.stride(1) == 1
    M, K = x.shape
    qs = max(K, pad_to or 0)
    xq = torch.empty((M, qs), dtype=torch.float8_e4m3fn, device=x.device)
    s = torch.empty((M, 1), dtype=torch.float32, device=x.device)
    check(_lib_().mi355_per_token_quant_fp8(xq.data_ptr(), s.data_ptr(), x.data_ptr(), M, K,
                                            x.stride(0), qs, _dt(x), _stream(x)), "per_token_quant_fp8")
    return xq, s


def fp8_scaled_mm(xq: torch.Tensor, wq: torch.Tensor, x_scale: torch.Tensor, w_scale: torch.Tensor,
                  out_dtype: torch.dtype, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp8_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype, bias) (sgl-kernel gemm.py) with
    wq given as [N, K] (one row per output channel)."""
    _gpu(xq, wq, x_scale, w_scale, bias)
    assert xq.is_contiguous() and wq.is_contiguous()
    M, K = xq.shape
    N = wq.shape[0]
    assert wq.shape[1] == K and x_scale.numel() == M and w_scale.numel() == N
    assert x_scale.dtype == torch.float32 and w_scale.dtype == torch.float32
    assert bias is None or bias.dtype == out_dtype
    y = torch.empty((M, N), dtype=out_dtype, device=xq.device)
    lib = _lib_()
    need = lib.mi355_fp8_workspace_bytes(M, N, K)
    ws = _workspace(xq.device, need, "fp8") if need > 0 else None
    check(lib.mi355_fp8_scaled_mm(y.data_ptr(), xq.data_ptr(), wq.data_ptr(), x_scale.data_ptr(),
                                  w_scale.data_ptr(), _p(bias), M, N, K, _p(ws),
                                  ws.numel() if ws is not None else 0, _DT[out_dtype],
                                  _stream(xq)), "fp8_scaled_mm")
    return y


def fp8_scaled_mm_tiled_supported(m: int, n: int, k: int, out_dtype: torch.dtype, silu_mul: bool = False) -> bool:
    """Whether fp8_scaled_mm_tiled serves the shape (16-bit output, K % 128 == 0, K >= 256, N % 16 == 0)."""
    return out_dtype in (torch.bfloat16, torch.float16) and bool(
        _lib_().mi355_fp8_scaled_mm_tiled_supported(m, n, k, _DT[out_dtype], 1 if silu_mul else 0))


def fp8_scaled_mm_tiled(xq: torch.Tensor, wq: torch.Tensor, x_scale: torch.Tensor, w_scale: torch.Tensor,
                        out_dtype: torch.dtype, bias: Optional[torch.Tensor] = None,
                        silu_mul: bool = False) -> torch.Tensor:
    """fp8_scaled_mm at prefill sizes on the 256 x 256-tile matrix-core kernel (wq [N, K]);
    silu_mul=True applies SiluAndMul to the [gate; up] output in the epilogue and returns [M, N / 2]."""
    _gpu(xq, wq, x_scale, w_scale, bias)
    assert xq.is_contiguous() and wq.is_contiguous()
    assert xq.dtype == torch.float8_e4m3fn and wq.dtype == torch.float8_e4m3fn
    M, K = xq.shape
    N = wq.shape[0]
    assert wq.shape[1] == K and x_scale.numel() == M and w_scale.numel() == N
    assert x_scale.dtype == torch.float32 and w_scale.dtype == torch.float32
    assert x_scale.is_contiguous() and w_scale.is_contiguous()
    assert bias is None or bias.dtype == out_dtype
    y = torch.empty((M, N // 2 if silu_mul else N), dtype=out_dtype, device=xq.device)
    if M == 0:
        return y
    check(_lib_().mi355_fp8_scaled_mm_tiled(y.data_ptr(), xq.data_ptr(), wq.data_ptr(), x_scale.data_ptr(),
                                            w_scale.data_ptr(), _p(bias), M, N, K, _DT[out_dtype],
                                            1 if silu_mul else 0, _stream(xq)), "fp8_scaled_mm_tiled")
    return y


def pack_weight_fp8(wq: torch.Tensor) -> torch.Tensor:
    """[N, K] e4m3fn weight -> packed copy for fp8_scaled_mm_packed (same 16-byte-fragment layout
    as pack_weight: the bytes are packed as an [N, K/2] 16-bit matrix)."""
    assert wq.dtype == torch.float8_e4m3fn and wq.is_contiguous() and wq.shape[1] % 64 == 0
    return pack_weight(wq.view(torch.bfloat16)).view(torch.float8_e4m3fn)


def fp8_scaled_mm_packed(xq: torch.Tensor, wq_packed: torch.Tensor, n: int, x_scale: torch.Tensor,
                         w_scale: torch.Tensor, out_dtype: torch.dtype,
                         bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp8_scaled_mm for M <= 64 on a weight from pack_weight_fp8 (n output features)."""
    _gpu(xq, wq_packed, x_scale, w_scale, bias)
    M, K = xq.shape
    assert xq.is_contiguous() and xq.dtype == torch.float8_e4m3fn and wq_packed.dtype == torch.float8_e4m3fn
    assert x_scale.dtype == torch.float32 and x_scale.numel() == M and w_scale.dtype == torch.float32
    assert w_scale.numel() == n and (bias is None or bias.dtype == out_dtype)
    y = torch.empty((M, n), dtype=out_dtype, device=xq.device)
    if M == 0:
        return y
    lib = _lib_()
    need = lib.mi355_fp8_packed_workspace_bytes(M, n, K)
    ws = _workspace(xq.device, need) if need > 0 else None
    check(lib.mi355_fp8_scaled_mm_packed(y.data_ptr(), xq.data_ptr(), wq_packed.data_ptr(), x_scale.data_ptr(),
                                         w_scale.data_ptr(), _p(bias), M, n, K, _p(ws),
                                         ws.numel() if ws is not None else 0, _DT[out_dtype], _stream(xq)),
          "fp8_scaled_mm_packed")
    return y


# ---------------------------------------------------------------------------------- sampling
def argmax(logits: torch.Tensor) -> torch.Tensor:
    """torch.argmax(logits, -1) on fp32 [B, V] (layers/sampler.py:74)."""
    _gpu(logits)
    assert logits.dim() == 2 and logits.dtype == torch.float32 and logits.stride(1) == 1
    ids = torch.empty(logits.shape[0], dtype=torch.int64, device=logits.device)
    rows = logits.shape[0]
    if 0 < rows < 256:
        # few rows: several workgroups per row (mi355_argmax_chunked); its cells live in a persistent zeroed workspace
        lib = _lib_()
        need = lib.mi355_argmax_workspace_bytes(rows)
        ws = _workspace(logits.device, need, tag="argmax")
        check(lib.mi355_argmax_chunked(ids.data_ptr(), logits.data_ptr(), rows, logits.shape[1], logits.stride(0),
                                       ws.data_ptr(), ws.numel(), _stream(logits)), "argmax_chunked")
        return ids
    check(_lib_().mi355_argmax(ids.data_ptr(), logits.data_ptr(), logits.shape[0], logits.shape[1],
                               logits.stride(0), _stream(logits)), "argmax")
    return ids


def softmax_temperature_(logits: torch.Tensor, temperatures: torch.Tensor) -> torch.Tensor:
    """In place logits.div_(temperatures); logits[:] = softmax(logits) (layers/sampler.py:79-81)."""
    _gpu(logits, temperatures)
    assert logits.dim() == 2 and logits.dtype == torch.float32 and logits.stride(1) == 1
    assert temperatures.dtype == torch.float32 and temperatures.numel() == logits.shape[0]
    check(_lib_().mi355_softmax_temperature(logits.data_ptr(), temperatures.data_ptr(),
                                            logits.shape[0], logits.shape[1], logits.stride(0),
                                            _stream(logits)), "softmax_temperature")
    return logits


def top_k_top_p_min_p_sample(probs: torch.Tensor, top_ks: Optional[torch.Tensor],
                             top_ps: Optional[torch.Tensor], min_ps: Optional[torch.Tensor],
                             uniform: torch.Tensor) -> torch.Tensor:
    """Joint top-k/top-p/min-p sampling from probabilities with caller-supplied uniforms."""
    _gpu(probs, top_ks, top_ps, min_ps, uniform)
    assert probs.dim() == 2 and probs.dtype == torch.float32 and probs.stride(1) == 1
    B = probs.shape[0]
    assert uniform.dtype == torch.float32 and uniform.numel() == B
    assert top_ks is None or (top_ks.dtype == torch.int32 and top_ks.numel() == B)
    assert top_ps is None or (top_ps.dtype == torch.float32 and top_ps.numel() == B)
    assert min_ps is None or (min_ps.dtype == torch.float32 and min_ps.numel() == B)
    ids = torch.empty(B, dtype=torch.int32, device=probs.device)
    check(_lib_().mi355_top_k_top_p_min_p_sample(ids.data_ptr(), probs.data_ptr(), _p(top_ks),
                                                 _p(top_ps), _p(min_ps), uniform.data_ptr(), B,
                                                 probs.shape[1], probs.stride(0), _stream(probs)),
          "top_k_top_p_min_p_sample")
    return ids


# ------------------------------------------------------- fp32 residual stream with per-sequence state
def _seg(tok_req, seg_start, seg_len):
    assert (tok_req is None) == (seg_start is None) == (seg_len is None), "tok_req, seg_start and seg_len come together"
    for t in (tok_req, seg_start, seg_len):
        assert t is None or (t.dtype == torch.int32 and t.is_contiguous())
    return _p(tok_req), _p(seg_start), _p(seg_len)


def bigram_embedding(ids: torch.Tensor, table: torch.Tensor, bigram: torch.Tensor, prev_token: torch.Tensor,
                     req_to_state: torch.Tensor, req_pool_indices: torch.Tensor, positions: torch.Tensor, scale: float,
                     mul_prev: int, mul_cur: int, buckets: int, tok_req=None, seg_start=None, seg_len=None) -> torch.Tensor:
    """fp32 [T, D]: table[id] * scale + bigram[(prev * mul_prev + id * mul_cur) % buckets] (row `buckets` at position 0);
    prev comes from the batch or, for a segment's first token, from prev_token[state slot]."""
    _gpu(ids, table, bigram, prev_token, req_to_state, req_pool_indices, positions)
    assert ids.dtype == torch.int64 and positions.dtype == torch.int64 and req_pool_indices.dtype == torch.int64
    assert prev_token.dtype == torch.int32 and req_to_state.dtype == torch.int32
    assert table.is_contiguous() and bigram.is_contiguous() and table.dtype == bigram.dtype
    assert bigram.shape == (buckets + 1, table.shape[1]) and ids.is_contiguous() and positions.is_contiguous()
    T, D = ids.numel(), table.shape[1]
    x = torch.empty((T, D), dtype=torch.float32, device=ids.device)
    tr, ss, sl = _seg(tok_req, seg_start, seg_len)
    check(_lib_().mi355_bigram_embedding(x.data_ptr(), ids.data_ptr(), table.data_ptr(), bigram.data_ptr(), prev_token.data_ptr(),
                                         req_to_state.data_ptr(), req_pool_indices.data_ptr(), tr, ss, sl, positions.data_ptr(),
                                         T, D, table.shape[0], float(scale), int(mul_prev), int(mul_cur), int(buckets),
                                         _dt(table), _stream(ids)), "bigram_embedding")
    return x


def layernorm_shift(x: torch.Tensor, weight: torch.Tensor, eps: float, shift: Optional[torch.Tensor] = None, state=None,
                    req_to_state=None, req_pool_indices=None, positions=None, h_last=None, tok_req=None, seg_start=None,
                    seg_len=None):
    """Weight-only layer norm of the fp32 rows x [T, D] -> h (weight's dtype).  With `shift` also the token-shifted rows
    hs = h + (h_prev - h) * shift; returns h or (h, hs).  h_last [B, D] fp32 receives the h of every segment's last token."""
    _gpu(x, weight, shift, state, req_to_state, req_pool_indices, positions, h_last)
    assert x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous() and weight.is_contiguous()
    T, D = x.shape
    assert weight.numel() == D
    h = torch.empty((T, D), dtype=weight.dtype, device=x.device)
    hs = None
    if shift is not None:
        assert shift.dtype == weight.dtype and shift.numel() == D and shift.is_contiguous()
        assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[-1] == D
        assert req_to_state.dtype == torch.int32 and req_pool_indices.dtype == torch.int64 and positions.dtype == torch.int64
        assert h_last is None or (h_last.dtype == torch.float32 and h_last.is_contiguous() and h_last.shape[-1] == D)
        hs = torch.empty_like(h)
    tr, ss, sl = _seg(tok_req, seg_start, seg_len)
    check(_lib_().mi355_layernorm_shift(h.data_ptr(), _p(hs), _p(h_last) if shift is not None else None, x.data_ptr(),
                                        weight.data_ptr(), _p(shift), _p(state), _p(req_to_state), _p(req_pool_indices),
                                        tr, ss, sl, _p(positions), T, D, float(eps), _dt(weight), _stream(x)), "layernorm_shift")
    return h if shift is None else (h, hs)


def commit_sequence_state(state: torch.Tensor, prev_token: Optional[torch.Tensor], h_last: torch.Tensor, ids: torch.Tensor,
                          req_to_state: torch.Tensor, req_pool_indices: torch.Tensor, seg_start=None, seg_len=None) -> None:
    """state [L, slots, D] <- h_last [L, B, D] at every sequence's slot; prev_token[slot] <- the segment's last token id."""
    _gpu(state, prev_token, h_last, ids, req_to_state, req_pool_indices)
    L, B, D = h_last.shape
    assert state.dim() == 3 and state.shape[0] == L and state.shape[2] == D and state.is_contiguous() and h_last.is_contiguous()
    assert state.dtype == torch.float32 and h_last.dtype == torch.float32 and ids.dtype == torch.int64
    assert req_pool_indices.numel() == B
    _, ss, sl = _seg(seg_start, seg_start, seg_len)
    check(_lib_().mi355_commit_sequence_state(state.data_ptr(), _p(prev_token), h_last.data_ptr(), ids.data_ptr(),
                                              req_to_state.data_ptr(), req_pool_indices.data_ptr(), ss, sl, B, L, D,
                                              state.stride(0), _stream(state)), "commit_sequence_state")


def gelu_tanh_and_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """gelu_tanh(gate) * up for two [T, d] column blocks of one projection output (equal row strides)."""
    _gpu(gate, up)
    assert gate.dim() == 2 and gate.shape == up.shape and gate.dtype == up.dtype
    assert gate.stride(1) == 1 and up.stride(1) == 1 and gate.stride(0) == up.stride(0)
    out = torch.empty(gate.shape, dtype=gate.dtype, device=gate.device)
    check(_lib_().mi355_gelu_tanh_and_mul(out.data_ptr(), gate.data_ptr(), up.data_ptr(), gate.shape[0], gate.shape[1],
                                          gate.stride(0), _dt(gate), _stream(gate)), "gelu_tanh_and_mul")
    return out


def gated_residual_add(x: torch.Tensor, g1: torch.Tensor, b1: torch.Tensor, y1: torch.Tensor, g2=None, b2=None, y2=None) -> None:
    """In place on the fp32 rows x: x += sigmoid(g1 + b1) * y1 (+ sigmoid(g2 + b2) * y2)."""
    _gpu(x, g1, b1, y1, g2, b2, y2)
    assert x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous()
    T, D = x.shape
    for t in (g1, y1, g2, y2):
        assert t is None or (t.shape == (T, D) and t.stride(1) == 1 and t.dtype == g1.dtype)
    assert b1.numel() == D and b1.dtype == g1.dtype and (g2 is None or g2.stride(0) == g1.stride(0))
    check(_lib_().mi355_gated_residual_add(x.data_ptr(), g1.data_ptr(), b1.data_ptr(), y1.data_ptr(), _p(g2), _p(b2), _p(y2), T, D,
                                           g1.stride(0), y1.stride(0), y2.stride(0) if y2 is not None else 0, _dt(g1),
                                           _stream(x)), "gated_residual_add")


# ------------------------------------------------------- windowed attention over a latent cache, softmax sink
def latent_norms_rope_write(a: torch.Tensor, q_weight: torch.Tensor, kv_weight: torch.Tensor, positions: torch.Tensor,
                            out_cache_loc: torch.Tensor, inv_freq: torch.Tensor, cache: torch.Tensor, q_rank: int, rank: int,
                            rope_dim: int, rot_dims: int, eps: float) -> torch.Tensor:
    """a [T, >= q_rank + rank + rope_dim]: returns cq = RMSnorm(a[:, :q_rank]) * q_weight and writes the cache rows
    [RMSnorm(kv latent) * kv_weight | rot(rope key)] at out_cache_loc."""
    _gpu(a, q_weight, kv_weight, positions, out_cache_loc, inv_freq, cache)
    assert a.dim() == 2 and a.stride(1) == 1 and cache.is_contiguous() and cache.dtype == a.dtype
    assert cache.shape[-1] == rank + rope_dim and q_weight.dtype == a.dtype == kv_weight.dtype
    assert q_weight.numel() == q_rank and kv_weight.numel() == rank
    assert inv_freq.dtype == torch.float32 and inv_freq.numel() >= rot_dims // 2
    assert positions.dtype == torch.int64 and out_cache_loc.dtype == torch.int64
    assert positions.is_contiguous() and out_cache_loc.is_contiguous()
    T = a.shape[0]
    cq = torch.empty((T, q_rank), dtype=a.dtype, device=a.device)
    check(_lib_().mi355_latent_norms_rope_write(cq.data_ptr(), cache.data_ptr(), a.data_ptr(), q_weight.data_ptr(),
                                                kv_weight.data_ptr(), positions.data_ptr(), out_cache_loc.data_ptr(),
                                                inv_freq.data_ptr(), T, a.stride(0), q_rank, rank, rope_dim, rot_dims,
                                                cache.shape[0], float(eps), _dt(a), _stream(a)), "latent_norms_rope_write")
    return cq


def latent_window_attention_block_tokens(heads: int, rank: int, rope_dim: int, dtype: torch.dtype) -> int:
    """Most consecutive tokens of one sequence that a workgroup of latent_window_attention takes (0: shape not served)."""
    return int(_lib_().mi355_latent_window_attention_block_tokens(heads, rank, rope_dim, _DT[dtype]))


def latent_window_attention_splits(tokens: int, heads: int, rank: int, window: int, max_position: int, dtype: torch.dtype) -> int:
    """Key ranges per token for a decode-sized launch of the 16-bit kernel: enough workgroups to cover the chip twice,
    at least 128 keys each."""
    if dtype not in (torch.bfloat16, torch.float16) or rank > 512:
        return 1
    keys = min(window, max_position + 1)
    wgs = max(1, tokens * ((heads + 63) // 64))
    return int(max(1, min(64, (512 + wgs - 1) // wgs, keys // 128)))


def latent_window_attention(qa: torch.Tensor, qr: torch.Tensor, cache: torch.Tensor, out: torch.Tensor, req_to_token: torch.Tensor,
                            req_pool_indices: torch.Tensor, positions: torch.Tensor, sink: torch.Tensor, inv_freq: torch.Tensor,
                            rot_dims: int, window: int, scale: float, gate: Optional[torch.Tensor] = None, tok_req=None,
                            blocks=None, num_splits: int = 1) -> torch.Tensor:
    """qa [T, H, rank] and out [T, H, rank] (any token / head strides), qr [T, H, rope_dim] unrotated, cache
    [slots, rank + rope_dim], gate [T, H] logits (row-strided) or None, blocks int32 [n, 2] runs of tokens or None."""
    _gpu(qa, qr, cache, out, req_to_token, req_pool_indices, positions, sink, inv_freq, gate, tok_req, blocks)
    T, H, rank = qa.shape
    rope_dim = cache.shape[-1] - rank
    assert out.shape == qa.shape and qa.stride(2) == 1 and out.stride(2) == 1 and cache.is_contiguous()
    assert qa.dtype == out.dtype == cache.dtype and sink.dtype == torch.float32 and sink.numel() == H and sink.is_contiguous()
    assert req_to_token.dtype == torch.int32 and req_pool_indices.dtype == torch.int64 and positions.dtype == torch.int64
    if rope_dim:
        assert qr.shape == (T, H, rope_dim) and qr.stride(2) == 1 and qr.dtype == qa.dtype and inv_freq.dtype == torch.float32
    assert gate is None or (gate.shape == (T, H) and gate.stride(1) == 1 and gate.dtype == qa.dtype)
    assert tok_req is None or (tok_req.dtype == torch.int32 and tok_req.numel() == T)
    if blocks is not None:
        assert blocks.dtype == torch.int32 and blocks.dim() == 2 and blocks.shape[1] == 2 and blocks.is_contiguous()
        nb = blocks.shape[0]
    else:
        nb = T
    scratch = None
    if num_splits > 1:
        assert blocks is None, "key splits serve launches of one token per run"
        scratch = torch.empty(num_splits * T * H * (rank + 2), dtype=torch.float32, device=qa.device)
    check(_lib_().mi355_latent_window_attention(
        out.data_ptr(), qa.data_ptr(), _p(qr) if rope_dim else None, cache.data_ptr(), _p(gate), req_to_token.data_ptr(),
        req_pool_indices.data_ptr(), _p(tok_req), positions.data_ptr(), _p(blocks), nb, sink.data_ptr(), _p(inv_freq),
        qa.stride(0), qa.stride(1), qr.stride(0) if rope_dim else 0, qr.stride(1) if rope_dim else 0, out.stride(0), out.stride(1),
        gate.stride(0) if gate is not None else 0, req_to_token.stride(0), H, rank, rope_dim, rot_dims, int(window), float(scale),
        int(num_splits), _p(scratch), T, _dt(qa), _stream(qa)), "latent_window_attention")
    return out


# ------------------------------------------------------- post-norm fp32 stream, head norms and rotations
def scaled_add_group_rmsnorm(x: torch.Tensor, branch: Optional[torch.Tensor], alpha: float, weight: torch.Tensor, groups: int,
                             eps: float, rows: Optional[torch.Tensor] = None, coef: Optional[torch.Tensor] = None,
                             inplace: bool = True) -> torch.Tensor:
    """y = N(alpha * x + branch) * weight, N the RMS norm over `groups` equal parts of the row.  inplace: x <- y; returns y
    in the weight's dtype (x itself for an fp32 model).  rows int32 [T, n] / coef fp32 [T, n]: token t's branch is
    sum_j coef[t, j] * branch[rows[t, j]]."""
    _gpu(x, branch, weight, rows, coef)
    assert x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous() and weight.is_contiguous() and weight.numel() == x.shape[1]
    T, D = x.shape
    n_branch = 1
    if rows is not None:
        assert rows.dtype == torch.int32 and coef.dtype == torch.float32 and rows.shape == coef.shape and rows.shape[0] == T
        assert rows.is_contiguous() and coef.is_contiguous() and branch is not None
        n_branch = rows.shape[1]
    if branch is not None:
        assert branch.dim() == 2 and branch.shape[1] == D and branch.stride(1) == 1 and branch.dtype == weight.dtype
        assert rows is not None or branch.shape[0] == T
    same = weight.dtype == torch.float32
    h = None if (same and inplace) else torch.empty((T, D), dtype=weight.dtype, device=x.device)
    check(_lib_().mi355_scaled_add_group_rmsnorm(x.data_ptr() if inplace else None, _p(h), x.data_ptr(), _p(branch),
                                                 branch.stride(0) if branch is not None else 0, _p(rows), _p(coef), n_branch,
                                                 float(alpha), weight.data_ptr(), T, D, int(groups), float(eps), _dt(weight),
                                                 _stream(x)), "scaled_add_group_rmsnorm")
    return x if h is None else h


def rmsnorm_residual_add(x: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float, offset: float = 0.0,
                         layer_scale: Optional[torch.Tensor] = None, mult: float = 1.0) -> torch.Tensor:
    """x += mult * layer_scale * y / sqrt(mean(y^2) + eps) * (offset + weight) in place on the fp32 rows (layer_scale [D] or
    None); returns the new x in the weight's dtype."""
    _gpu(x, y, weight, layer_scale)
    assert x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous() and y.shape == x.shape and y.stride(1) == 1
    assert y.dtype == weight.dtype and weight.is_contiguous() and weight.numel() == x.shape[1]
    assert layer_scale is None or (layer_scale.dtype == weight.dtype and layer_scale.is_contiguous() and layer_scale.numel() == x.shape[1])
    T, D = x.shape
    h = None if weight.dtype == torch.float32 else torch.empty((T, D), dtype=weight.dtype, device=x.device)
    check(_lib_().mi355_rmsnorm_residual_add_scaled(x.data_ptr(), _p(h), y.data_ptr(), y.stride(0), weight.data_ptr(), _p(layer_scale),
                                                    float(offset), float(mult), T, D, float(eps), _dt(weight), _stream(x)),
          "rmsnorm_residual_add")
    return x if h is None else h


def gated_group_rmsnorm(y: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    """fp32 rows y [T, D], gate [T, D] (row-strided, the weight's dtype) -> N(y * silu(gate)) * weight with N the RMS norm over
    `groups` equal consecutive parts of the row: gated first, normed after.  Result in the weight's dtype."""
    _gpu(y, gate, weight)
    T, D = y.shape
    assert y.dtype == torch.float32 and y.is_contiguous() and gate.shape == (T, D) and gate.stride(1) == 1
    assert gate.dtype == weight.dtype and weight.is_contiguous() and weight.numel() == D and D % groups == 0
    out = torch.empty((T, D), dtype=weight.dtype, device=y.device)
    check(_lib_().mi355_gated_group_rmsnorm(out.data_ptr(), y.data_ptr(), gate.data_ptr(), gate.stride(0), weight.data_ptr(), T, D,
                                            int(groups), float(eps), _dt(weight), _stream(y)), "gated_group_rmsnorm")
    return out


def head_norm_rope(src: torch.Tensor, weight: Optional[torch.Tensor], eps: float, positions: torch.Tensor, inv_freq: torch.Tensor,
                   rot_dims: int, interleaved: bool, scale: float, out_dtype: torch.dtype, cache: Optional[torch.Tensor] = None,
                   loc: Optional[torch.Tensor] = None, rot_mag: float = 1.0) -> torch.Tensor:
    """src [T, H, d] (token / head strides free) -> optional RMS norm per head, rotation of the first rot_dims features (cos
    and sin times rot_mag), scale; to a new [T, H, d] tensor of out_dtype, or into cache[loc[t]] ([slots, H, d]) when a cache
    is given."""
    _gpu(src, weight, positions, inv_freq, cache, loc)
    T, H, d = src.shape
    assert src.stride(2) == 1 and positions.dtype == torch.int64 and positions.is_contiguous()
    assert weight is None or (weight.dtype == src.dtype and weight.numel() == d and weight.is_contiguous())
    assert rot_dims == 0 or (inv_freq.dtype == torch.float32 and inv_freq.numel() >= rot_dims // 2)
    if cache is not None:
        assert cache.is_contiguous() and cache.shape[1:] == (H, d) and loc is not None and loc.dtype == torch.int64
        assert loc.is_contiguous() and loc.numel() == T
        out, out_dtype = cache, cache.dtype
    else:
        out = torch.empty((T, H, d), dtype=out_dtype, device=src.device)
        loc = None
    check(_lib_().mi355_head_norm_rope_mag(out.data_ptr(), src.data_ptr(), _p(weight), positions.data_ptr(), _p(loc),
                                           _p(inv_freq) if rot_dims else None, T, H, d, src.stride(0), src.stride(1), out.stride(0),
                                           out.stride(1), out.shape[0], int(rot_dims), int(bool(interleaved)), float(scale),
                                           float(eps), float(rot_mag), _dt(src), _DT[out_dtype], _stream(src)), "head_norm_rope")
    return out


def qkv_norm_rope_write(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, wq: torch.Tensor, wk: torch.Tensor, eps: float,
                        positions: torch.Tensor, inv_freq: Optional[torch.Tensor], rot_dims: int, interleaved: bool, rot_mag: float,
                        k_cache: torch.Tensor, v_cache: torch.Tensor, loc: torch.Tensor) -> torch.Tensor:
    """The three head norms of an attention layer in one launch: q [T, H, d], k [T, G, d], v [T, G, dv] (column blocks of one
    projection's output will do).  Returns head_norm_rope(q, wq, ...) as a new [T, H, d]; head_norm_rope(k, wk, ...) goes into
    k_cache[loc], v / rms(v) into v_cache[loc]."""
    _gpu(q, k, v, wq, wk, positions, inv_freq, k_cache, v_cache, loc)
    T, H, d = q.shape
    G, dv = k.shape[1], v.shape[2]
    assert k.shape == (T, G, d) and v.shape == (T, G, dv) and q.dtype == k.dtype == v.dtype == k_cache.dtype == v_cache.dtype
    for t_ in (q, k, v):
        assert t_.stride(2) == 1 and t_.stride(1) == t_.shape[2], "heads lie side by side in a token's row"
    assert wq.dtype == q.dtype and wk.dtype == q.dtype and wq.numel() == d and wk.numel() == d and wq.is_contiguous() and wk.is_contiguous()
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.shape[1:] == (G, d) and v_cache.shape[1:] == (G, dv)
    assert positions.dtype == torch.int64 and positions.is_contiguous() and loc.dtype == torch.int64 and loc.is_contiguous() and loc.numel() == T
    assert rot_dims == 0 or (inv_freq.dtype == torch.float32 and inv_freq.numel() >= rot_dims // 2)
    out = torch.empty((T, H, d), dtype=q.dtype, device=q.device)
    check(_lib_().mi355_qkv_norm_rope_write(out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                            q.stride(0), k.stride(0), v.stride(0), wq.data_ptr(), wk.data_ptr(), positions.data_ptr(),
                                            loc.data_ptr(), _p(inv_freq) if rot_dims else None, T, H, G, d, dv, int(rot_dims),
                                            int(bool(interleaved)), float(eps), float(rot_mag), _dt(q), _stream(q)), "qkv_norm_rope_write")
    return out


def head_rmsnorm_gate(o: torch.Tensor, weight: Optional[torch.Tensor], gate: torch.Tensor, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """o fp32 [T, H, dv] -> o / rms(o) (* weight) * silu(gate) as [T, H * dv] of the gate's dtype; gate [T, H * dv] row-strided."""
    _gpu(o, weight, gate)
    T, H, dv = o.shape
    assert o.dtype == torch.float32 and o.is_contiguous() and gate.shape == (T, H * dv) and gate.stride(1) == 1
    assert gate.dtype == out_dtype and (weight is None or (weight.dtype == out_dtype and weight.numel() == dv and weight.is_contiguous()))
    out = torch.empty((T, H * dv), dtype=out_dtype, device=o.device)
    check(_lib_().mi355_head_rmsnorm_gate(out.data_ptr(), o.data_ptr(), _p(weight), gate.data_ptr(), gate.stride(0), T, H, dv,
                                          float(eps), _dt(gate), _stream(o)), "head_rmsnorm_gate")
    return out


def gelu_tanh_mul_rows(gate: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, col_off: int) -> torch.Tensor:
    """gelu_tanh(gate [T, d]) * table[ids, col_off: col_off + d]."""
    _gpu(gate, table, ids)
    T, d = gate.shape
    assert gate.stride(1) == 1 and table.dim() == 2 and table.stride(1) == 1 and table.dtype == gate.dtype
    assert ids.dtype == torch.int64 and ids.is_contiguous() and ids.numel() == T and 0 <= col_off and col_off + d <= table.shape[1]
    out = torch.empty((T, d), dtype=gate.dtype, device=gate.device)
    check(_lib_().mi355_gelu_tanh_mul_rows(out.data_ptr(), gate.data_ptr(), gate.stride(0), table.data_ptr(), table.shape[0],
                                           table.stride(0), int(col_off), ids.data_ptr(), T, d, _dt(gate), _stream(gate)),
          "gelu_tanh_mul_rows")
    return out


# ------------------------------------------------------- linear recurrence over per-sequence matrices
def linear_recurrence(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor, state: torch.Tensor,
                      req_to_state: torch.Tensor, req_pool_indices: torch.Tensor, positions: torch.Tensor, q_scale: float,
                      gate_logits: Optional[torch.Tensor] = None, gate_bias: Optional[torch.Tensor] = None, tau: float = 1.0,
                      head_decay: Optional[torch.Tensor] = None, tok_req=None, seg_start=None, seg_len=None,
                      dt_logits: Optional[torch.Tensor] = None, dt_bias: Optional[torch.Tensor] = None,
                      rate_log: Optional[torch.Tensor] = None, skip: Optional[torch.Tensor] = None) -> torch.Tensor:
    """S = diag(a) S + k v^T, out = S^T (q * q_scale) per head over every sequence's tokens of the step, on
    state[slot] ([slots, H, dk, dv] fp32, read unless the sequence starts at position 0, written back).  q, k [T, H, dk]
    (fp32 or v's dtype), v [T, H, dv]; the decay from gate_logits fp32 [T, H * dk] (+ gate_bias, / tau) or head_decay fp32 [H],
    or (state-space form) from step sizes: dt = softplus(dt_logits [T, H] + dt_bias [H]), a = exp(-exp(rate_log [H]) dt),
    S = a S + dt k v^T, out += skip [H] * v (all fp32).  q and k may have G < H heads (head h reads head h // (H / G))."""
    _gpu(q, k, v, out, state, req_to_state, req_pool_indices, positions, gate_logits, gate_bias, head_decay, dt_logits, dt_bias,
         rate_log, skip)
    T, G, dk = q.shape
    H, dv = v.shape[1], v.shape[2]
    assert k.shape == q.shape and v.shape[0] == T and H % G == 0 and q.dtype == k.dtype and q.dtype in (v.dtype, torch.float32)
    for t in (q, k, v):
        assert t.stride(2) == 1 and t.stride(1) == t.shape[2], "heads lie side by side in a token's row"
    assert out.dtype == torch.float32 and out.shape == (T, H, dv) and out.is_contiguous()
    assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, dk, dv)
    assert req_to_state.dtype == torch.int32 and req_pool_indices.dtype == torch.int64 and positions.dtype == torch.int64
    assert (gate_logits is not None) + (head_decay is not None) + (dt_logits is not None) == 1
    if dt_logits is not None:
        assert dt_logits.dtype == torch.float32 and dt_logits.shape == (T, H) and dt_logits.stride(1) == 1
        for w in (dt_bias, rate_log, skip):
            assert w is None or (w.dtype == torch.float32 and w.numel() == H and w.is_contiguous())
        assert dt_bias is not None and rate_log is not None
    elif gate_logits is not None:
        assert gate_logits.dtype == torch.float32 and gate_logits.shape == (T, H * dk) and gate_logits.stride(1) == 1
        assert gate_bias is None or (gate_bias.dtype == v.dtype and gate_bias.numel() == H * dk and gate_bias.is_contiguous())
    else:
        assert head_decay.dtype == torch.float32 and head_decay.numel() == H and head_decay.is_contiguous()
    _, ss, sl = _seg(tok_req, seg_start, seg_len)
    B = req_pool_indices.numel()
    assert seg_start is not None or B == T, "without segments every token is a sequence of its own"
    check(_lib_().mi355_linear_recurrence_ssm(out.data_ptr(), state.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                              _p(gate_logits), _p(gate_bias), _p(head_decay), _p(dt_logits),
                                              dt_logits.stride(0) if dt_logits is not None else 0, _p(dt_bias), _p(rate_log), _p(skip),
                                              req_to_state.data_ptr(), req_pool_indices.data_ptr(), ss, sl, positions.data_ptr(), B,
                                              H, G, dk, dv, q.stride(0), k.stride(0), v.stride(0),
                                              gate_logits.stride(0) if gate_logits is not None else 0, float(q_scale), float(tau),
                                              _dt(q), _dt(v), _stream(q)), "linear_recurrence")
    return out


# ------------------------------------------------------- causal attention with sigmoid weights
def sigmoid_attention_block_tokens(heads: int, kv_heads: int, head_dim: int, v_head_dim: int, dtype: torch.dtype) -> int:
    """Most consecutive tokens of one sequence that a workgroup of sigmoid_attention takes."""
    return int(_lib_().mi355_sigmoid_attention_block_tokens(heads, kv_heads, head_dim, v_head_dim, _DT[dtype]))


def sigmoid_attention_splits(tokens: int, heads: int, kv_heads: int, max_len: int, dtype: torch.dtype) -> int:
    """Key ranges per token for a decode-sized launch: eight workgroups per CU in flight (a workgroup waits on its own
    loads; its neighbours' products cover them), at least 128 keys each."""
    wgs = max(1, tokens * kv_heads * ((heads // kv_heads + 63) // 64))
    return int(max(1, min(64, (2048 + wgs - 1) // wgs, max_len // 128)))


def sigmoid_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor, req_to_token: torch.Tensor,
                      req_pool_indices: torch.Tensor, positions: torch.Tensor, temp: torch.Tensor, bias: torch.Tensor, scale: float,
                      tok_req=None, blocks=None, num_splits: int = 1, max_run: Optional[int] = None) -> torch.Tensor:
    """q [T, H, d], caches [slots, G, d] / [slots, G, dv], out [T, H, dv]; temp / bias fp32 [H]; blocks int32 [n, 2] runs of
    at most max_run consecutive tokens of one sequence, or None (one token per run)."""
    _gpu(q, k_cache, v_cache, out, req_to_token, req_pool_indices, positions, temp, bias, tok_req, blocks)
    T, H, d = q.shape
    G, dv = k_cache.shape[1], v_cache.shape[2]
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.shape[2] == d and v_cache.shape[1] == G
    assert out.shape == (T, H, dv) and q.stride(2) == 1 and out.stride(2) == 1 and q.dtype == out.dtype == k_cache.dtype == v_cache.dtype
    assert temp.dtype == torch.float32 and bias.dtype == torch.float32 and temp.numel() == H and bias.numel() == H
    assert temp.is_contiguous() and bias.is_contiguous()
    assert req_to_token.dtype == torch.int32 and req_pool_indices.dtype == torch.int64 and positions.dtype == torch.int64
    assert tok_req is None or (tok_req.dtype == torch.int32 and tok_req.numel() == T)
    if blocks is not None:
        assert blocks.dtype == torch.int32 and blocks.dim() == 2 and blocks.shape[1] == 2 and blocks.is_contiguous()
        nb, num_splits = blocks.shape[0], 1
        assert max_run is not None, "runs come with their longest length"
    else:
        nb, max_run = T, 1
    scratch = torch.empty(num_splits * T * H * dv, dtype=torch.float32, device=q.device) if num_splits > 1 else None
    check(_lib_().mi355_sigmoid_attention(
        out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), req_to_token.data_ptr(), req_pool_indices.data_ptr(),
        _p(tok_req), positions.data_ptr(), _p(blocks), nb, temp.data_ptr(), bias.data_ptr(), q.stride(0), q.stride(1),
        out.stride(0), out.stride(1), req_to_token.stride(0), H, G, d, dv, float(scale), int(num_splits), _p(scratch), T,
        int(max_run), _dt(q), _stream(q)), "sigmoid_attention")
    return out


# ------------------------------------------------------- mixture of experts
def moe_route_grouped(logits: torch.Tensor, correction: torch.Tensor, top: int, n_groups: int, keep_groups: int,
                      scale: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """fp32 logits [T, E] -> (expert ids int32 [T, top], weights fp32 [T, top])."""
    _gpu(logits, correction)
    T, E = logits.shape
    assert logits.dtype == torch.float32 and logits.is_contiguous() and correction.dtype == torch.float32 and correction.numel() == E
    ids = torch.empty((T, top), dtype=torch.int32, device=logits.device)
    w = torch.empty((T, top), dtype=torch.float32, device=logits.device)
    check(_lib_().mi355_moe_route_grouped(ids.data_ptr(), w.data_ptr(), logits.data_ptr(), correction.data_ptr(), T, E, int(top),
                                          int(n_groups), int(keep_groups), float(scale), _stream(logits)), "moe_route_grouped")
    return ids, w


class MoePlan:
    """The sorted layout of a step's (token, expert) pairs, all on the device: src_row int32 [padded] (token of a sorted
    row, -1 for padding), rows int32 [T, top] (sorted row of a pair), tile_expert int32 [padded / block], n_tiles int32 [1]."""
    __slots__ = ("src_row", "rows", "tile_expert", "n_tiles", "block", "padded")

    def __init__(self, src_row, rows, tile_expert, n_tiles, block, padded):
        self.src_row, self.rows, self.tile_expert, self.n_tiles, self.block, self.padded = src_row, rows, tile_expert, n_tiles, block, padded


ROUTER_SKINNY_MAX_ROWS = 256


def moe_router_logits(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """fp32 x [T, D] against the fp32 router table [E, D] -> exact fp32 logits [T, E].  Few rows go to a wave-per-row kernel
    (a tiled GEMM with E columns would occupy a handful of CUs), many to the exact tiled GEMM."""
    _gpu(x, weight)
    assert x.dtype == torch.float32 and weight.dtype == torch.float32 and x.is_contiguous() and weight.is_contiguous()
    T, K = x.shape
    if T > ROUTER_SKINNY_MAX_ROWS or K > 16384:
        return linear(x, weight)
    out = torch.empty((T, weight.shape[0]), dtype=torch.float32, device=x.device)
    check(_lib_().mi355_moe_router_logits(out.data_ptr(), x.data_ptr(), weight.data_ptr(), T, weight.shape[0], K, _stream(x)),
          "moe_router_logits")
    return out


def moe_align(expert_ids: torch.Tensor, num_experts: int, wide_ok: bool = False, tiled_ok: bool = False) -> MoePlan:
    """wide_ok: the grouped GEMMs that follow can take blocks of 128 rows (16-bit operands, 16-byte rows); tiled_ok: they
    can run on the prefill projection kernel over blocks of 256 rows (linear_tiled_supported for both of them).  The
    larger blocks are used when the experts have at least two of them worth of rows on average."""
    _gpu(expert_ids)
    T, top = expert_ids.shape
    assert expert_ids.dtype == torch.int32 and expert_ids.is_contiguous()
    wide = 2 if (tiled_ok and T * top >= 512 * num_experts) else 1 if ((wide_ok or tiled_ok) and T * top >= 256 * num_experts) else 0
    block = int(_lib_().mi355_moe_block_rows(wide))
    pairs = T * top
    padded = (pairs + min(num_experts, pairs) * (block - 1) + block - 1) // block * block
    dev = expert_ids.device
    src_row = torch.empty(max(padded, 1), dtype=torch.int32, device=dev)
    rows = torch.empty((T, top), dtype=torch.int32, device=dev)
    tile_expert = torch.empty(max(padded // block, 1), dtype=torch.int32, device=dev)
    n_tiles = torch.empty(1, dtype=torch.int32, device=dev)
    check(_lib_().mi355_moe_align(src_row.data_ptr(), rows.data_ptr(), tile_expert.data_ptr(), n_tiles.data_ptr(),
                                  expert_ids.data_ptr(), T, top, int(num_experts), block, padded, _stream(expert_ids)), "moe_align")
    return MoePlan(src_row, rows, tile_expert, n_tiles, block, padded)


def moe_grouped_linear(x: torch.Tensor, w: torch.Tensor, plan: MoePlan, gather: bool, gelu: bool) -> torch.Tensor:
    """out [padded, N] = act(w[expert of the row's block] . x[src_row or the row itself]); rows of blocks not in use are
    left unwritten (nothing reads them)."""
    _gpu(x, w)
    E, N, K = w.shape
    assert w.is_contiguous() and x.dim() == 2 and x.shape[1] == K and x.stride(1) == 1 and x.dtype == w.dtype
    assert gather or x.shape[0] == plan.padded
    out = torch.empty((plan.padded, N), dtype=x.dtype, device=x.device)
    check(_lib_().mi355_moe_grouped_linear(out.data_ptr(), x.data_ptr(), x.stride(0), w.data_ptr(), plan.src_row.data_ptr(),
                                           plan.tile_expert.data_ptr(), plan.n_tiles.data_ptr(), int(gather), int(gelu),
                                           plan.padded, plan.block, N, K, _dt(x), _stream(x)), "moe_grouped_linear")
    return out


# ------------------------------------------------------- pre-norm fp32 stream with parallel branches
def offset_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, offset: float = 1.0) -> torch.Tensor:
    """fp32 rows x [T, D] -> x / sqrt(mean(x^2) + eps) * (offset + weight) in the weight's dtype (a weight stored around zero)."""
    _gpu(x, weight)
    assert x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous() and weight.is_contiguous() and weight.numel() == x.shape[1]
    T, D = x.shape
    h = torch.empty((T, D), dtype=weight.dtype, device=x.device)
    check(_lib_().mi355_offset_rmsnorm(h.data_ptr(), x.data_ptr(), weight.data_ptr(), T, D, float(eps), float(offset),
                                       _dt(weight), _stream(x)), "offset_rmsnorm")
    return h


def branch_residual_add(x: torch.Tensor, a: torch.Tensor, wa: Optional[torch.Tensor], b: Optional[torch.Tensor] = None,
                        wb: Optional[torch.Tensor] = None, s: float = 1.0, f: Optional[torch.Tensor] = None,
                        rows: Optional[torch.Tensor] = None, coef: Optional[torch.Tensor] = None, eps: float = 1e-6) -> torch.Tensor:
    """x += s * (A + B) + F in place on the fp32 rows: A = a / rms(a) * wa (wa None: a itself), B likewise from b, wb (b None:
    nothing), F = f, or sum_j coef[t, j] * f[rows[t, j]] (rows int32 [T, n], coef fp32 [T, n]), or nothing."""
    _gpu(x, a, wa, b, wb, f, rows, coef)
    assert x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous()
    T, D = x.shape
    n_branch = 1
    for y in (a, b):
        assert y is None or (y.shape == (T, D) and y.stride(1) == 1 and y.dtype == a.dtype)
    for w in (wa, wb):
        assert w is None or (w.dtype == a.dtype and w.numel() == D and w.is_contiguous())
    if f is not None:
        assert f.dim() == 2 and f.shape[1] == D and f.stride(1) == 1 and f.dtype == a.dtype
    if rows is not None:
        assert rows.dtype == torch.int32 and coef.dtype == torch.float32 and rows.shape == coef.shape and rows.shape[0] == T
        assert rows.is_contiguous() and coef.is_contiguous() and f is not None
        n_branch = rows.shape[1]
    else:
        assert f is None or f.shape[0] == T
    check(_lib_().mi355_branch_residual_add(x.data_ptr(), a.data_ptr(), a.stride(0), _p(wa), _p(b), b.stride(0) if b is not None else 0,
                                            _p(wb), float(s), _p(f), f.stride(0) if f is not None else 0, _p(rows), _p(coef),
                                            n_branch, T, D, float(eps), _dt(a), _stream(x)), "branch_residual_add")
    return x


def head_rmsnorm_gate_act(o: torch.Tensor, weight: Optional[torch.Tensor], gate: torch.Tensor, eps: float, out_dtype: torch.dtype,
                          gate_act: str = "silu") -> torch.Tensor:
    """head_rmsnorm_gate with the gate's function chosen: "silu" or "sigmoid"."""
    _gpu(o, weight, gate)
    T, H, dv = o.shape
    assert o.dtype == torch.float32 and o.is_contiguous() and gate.shape == (T, H * dv) and gate.stride(1) == 1
    assert gate.dtype == out_dtype and (weight is None or (weight.dtype == out_dtype and weight.numel() == dv and weight.is_contiguous()))
    out = torch.empty((T, H * dv), dtype=out_dtype, device=o.device)
    check(_lib_().mi355_head_rmsnorm_gate_act(out.data_ptr(), o.data_ptr(), _p(weight), gate.data_ptr(), gate.stride(0), T, H, dv,
                                              float(eps), {"silu": 0, "sigmoid": 1}[gate_act], _dt(gate), _stream(o)),
          "head_rmsnorm_gate")
    return out


ACTIVATIONS = {"none": 0, "silu": 1, "relu2": 2}


def causal_conv(u: torch.Tensor, w1: torch.Tensor, state: torch.Tensor, req_to_state: torch.Tensor, req_pool_indices: torch.Tensor,
                positions: torch.Tensor, w2: Optional[torch.Tensor] = None, residual: bool = False, act: str = "none",
                tok_req=None, seg_start=None, seg_len=None, bias: Optional[torch.Tensor] = None):
    """Causal convolution over time per channel of u [T, C] (row-strided) with filter w1 [C, taps] (last column: the current
    token) and, optionally, a second filter w2 over the same input; with `residual`, u is added to each result; then `act`.
    Inputs before a step's first token of a sequence come from state[slot] (fp32 [slots, taps - 1, C]; zeros before position
    0); afterwards the state holds the sequence's last taps - 1 inputs.  Returns y1, or (y1, y2)."""
    _gpu(u, w1, w2, state, req_to_state, req_pool_indices, positions, bias)
    T, C = u.shape
    taps = w1.shape[1]
    assert bias is None or (bias.dtype == u.dtype and bias.numel() == C and bias.is_contiguous()), "bias [C] of the first filter"
    assert u.stride(1) == 1 and w1.shape == (C, taps) and w1.is_contiguous() and w1.dtype == u.dtype
    assert w2 is None or (w2.shape == w1.shape and w2.is_contiguous() and w2.dtype == u.dtype)
    assert state.dtype == torch.float32 and state.is_contiguous() and tuple(state.shape[1:]) == (taps - 1, C)
    assert req_to_state.dtype == torch.int32 and req_pool_indices.dtype == torch.int64 and positions.dtype == torch.int64
    assert positions.is_contiguous() and positions.numel() == T
    y1 = torch.empty((T, C), dtype=u.dtype, device=u.device)
    y2 = torch.empty_like(y1) if w2 is not None else None
    tr, ss, sl = _seg(tok_req, seg_start, seg_len)
    assert seg_start is not None or req_pool_indices.numel() == T, "without segments every token is a sequence of its own"
    lib = _lib_()
    check(lib.mi355_causal_conv_bias(y1.data_ptr(), _p(y2), u.data_ptr(), u.stride(0), w1.data_ptr(), _p(w2), _p(bias),
                                     _p(state) if taps > 1 else None, req_to_state.data_ptr(), req_pool_indices.data_ptr(), tr, ss,
                                     positions.data_ptr(), T, C, taps, int(bool(residual)), ACTIVATIONS[act], _dt(u), _stream(u)),
          "causal_conv")
    if seg_start is not None and taps > 1:
        check(lib.mi355_causal_conv_state_update(state.data_ptr(), u.data_ptr(), u.stride(0), req_to_state.data_ptr(),
                                                 req_pool_indices.data_ptr(), ss, sl, positions.data_ptr(), req_pool_indices.numel(),
                                                 C, taps, _dt(u), _stream(u)), "causal_conv_state_update")
    return y1 if w2 is None else (y1, y2)


def activation(x: torch.Tensor, act: str) -> torch.Tensor:
    """act(x) over a row-strided [T, d] block, contiguous result: "silu" or "relu2" (the square of relu)."""
    _gpu(x)
    T, d = x.shape
    assert x.stride(1) == 1 and act in ("silu", "relu2")
    out = torch.empty((T, d), dtype=x.dtype, device=x.device)
    check(_lib_().mi355_activation(out.data_ptr(), x.data_ptr(), x.stride(0), T, d, ACTIVATIONS[act], _dt(x), _stream(x)), "activation")
    return out


def gated_delta_rule(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, beta_logits: torch.Tensor, gate_logits: torch.Tensor,
                     rate_bias: torch.Tensor, rate_log: torch.Tensor, out: torch.Tensor, state: torch.Tensor,
                     req_to_state: torch.Tensor, req_pool_indices: torch.Tensor, positions: torch.Tensor, q_scale: float,
                     tok_req=None, seg_start=None, seg_len=None) -> torch.Tensor:
    """Per head  S = diag(a) S;  u = beta (v - S^T k);  S += k u^T;  out = S^T (q * q_scale)  over every sequence's tokens of the
    step on state[slot] ([slots, H, dk, dv] fp32).  q, k [T, G, dk] (fp32 or v's dtype; head h reads head h // (H / G)), v
    [T, H, dv], beta_logits [T, H] (row-strided, v's dtype or fp32), gate_logits fp32 [T, H * dk], rate_bias fp32 [H * dk],
    rate_log fp32 [H]:  a = exp(-exp(rate_log) * softplus(gate_logits + rate_bias)),  beta = sigmoid(beta_logits).  With
    gate_logits [T, H] and rate_bias [H] the decay is one number per head and token."""
    _gpu(q, k, v, beta_logits, gate_logits, rate_bias, rate_log, out, state, req_to_state, req_pool_indices, positions)
    T, G, dk = q.shape
    H, dv = v.shape[1], v.shape[2]
    assert k.shape == q.shape and v.shape[0] == T and H % G == 0 and q.dtype == k.dtype and q.dtype in (v.dtype, torch.float32)
    for t in (q, k, v):
        assert t.stride(2) == 1 and t.stride(1) == t.shape[2], "heads lie side by side in a token's row"
    assert beta_logits.shape == (T, H) and beta_logits.stride(1) == 1 and beta_logits.dtype in (v.dtype, torch.float32)
    per_head = gate_logits.shape[1] == H and rate_bias.numel() == H
    assert gate_logits.dtype == torch.float32 and gate_logits.shape == (T, H if per_head else H * dk) and gate_logits.stride(1) == 1
    assert rate_bias.dtype == torch.float32 and rate_bias.numel() == (H if per_head else H * dk) and rate_bias.is_contiguous()
    assert rate_log.dtype == torch.float32 and rate_log.numel() == H and rate_log.is_contiguous()
    assert out.dtype == torch.float32 and out.shape == (T, H, dv) and out.is_contiguous()
    assert state.dtype == torch.float32 and state.is_contiguous() and tuple(state.shape[1:]) == (H, dk, dv)
    assert req_to_state.dtype == torch.int32 and req_pool_indices.dtype == torch.int64 and positions.dtype == torch.int64
    _, ss, sl = _seg(tok_req, seg_start, seg_len)
    B = req_pool_indices.numel()
    assert seg_start is not None or B == T, "without segments every token is a sequence of its own"
    check(_lib_().mi355_gated_delta_rule_ex(out.data_ptr(), state.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                            beta_logits.data_ptr(), gate_logits.data_ptr(), rate_bias.data_ptr(), rate_log.data_ptr(),
                                            req_to_state.data_ptr(), req_pool_indices.data_ptr(), ss, sl, positions.data_ptr(), B, H, G,
                                            dk, dv, q.stride(0), k.stride(0), v.stride(0), beta_logits.stride(0), gate_logits.stride(0),
                                            float(q_scale), int(per_head), int(beta_logits.dtype == torch.float32 and v.dtype != torch.float32),
                                            _dt(q), _dt(v), _stream(q)), "gated_delta_rule")
    return out


def window_attention_block_tokens(heads: int, kv_heads: int, head_dim: int, v_head_dim: int, dtype: torch.dtype) -> int:
    """Most consecutive tokens of one sequence that a workgroup of window_attention takes."""
    return int(_lib_().mi355_window_attention_block_tokens(heads, kv_heads, head_dim, v_head_dim, _DT[dtype]))


def window_attention_splits(tokens: int, heads: int, kv_heads: int, max_len: int, window: int, dtype: torch.dtype, pool: int = 0) -> int:
    """Key ranges per token for a decode-sized launch: two workgroups per CU, at least 256 visible keys each.  Measured on
    MI355X (64 sequences x 1024 keys, heads of 128): with 256 workgroups two ranges take 0.64 of one range's time, four 0.76,
    eight as long as one; with 512 workgroups one range is best -- every further range adds a workgroup's fixed cost (its
    query tile, its partial results and their merge) to a walk that is short already."""
    wgs = max(1, tokens * kv_heads * ((heads // kv_heads + 63) // 64))
    seen = min(max_len, window) if window > 0 else max_len
    if pool > 0 and window > 0:
        seen += max(0, max_len - window) // pool        # the averaged blocks before the window
    return int(max(1, min(64, 512 // wgs, seen // 256)))


def window_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor, req_to_token: torch.Tensor,
                     req_pool_indices: torch.Tensor, positions: torch.Tensor, sink: Optional[torch.Tensor], window: int, scale: float,
                     tok_req=None, blocks=None, max_run: Optional[int] = None, num_splits: int = 1, pool: int = 0,
                     pooled_k: Optional[torch.Tensor] = None, pooled_v: Optional[torch.Tensor] = None, pool_div: int = 1,
                     head_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Softmax attention of q [T, H, d] over the keys within `window` positions (0: all earlier ones) in caches
    [slots, G, d] / [slots, G, dv], with exp(sink[h]) added to the denominator (sink fp32 [H] or None) -> out [T, H, dv];
    blocks int32 [n, 2] runs of at most max_run consecutive tokens of one sequence, or None (one token per run).
    pool > 0: a token at position i also sees the averaged row of every block b of `pool` positions with
    b pool + pool - 1 <= i - window, at pooled_k / pooled_v [slot(b pool + pool - 1) // pool_div].  head_gate [T, H]
    (row-strided logits): head h's result times their sigmoid."""
    _gpu(q, k_cache, v_cache, out, req_to_token, req_pool_indices, positions, sink, tok_req, blocks, pooled_k, pooled_v, head_gate)
    if pool > 0:
        assert window > 0 and pooled_k is not None and pooled_v is not None and pool_div in (1, pool)
        assert pooled_k.is_contiguous() and pooled_v.is_contiguous() and pooled_k.dtype == pooled_v.dtype == k_cache.dtype
        assert pooled_k.shape[1:] == k_cache.shape[1:] and pooled_v.shape[1:] == v_cache.shape[1:]
    assert head_gate is None or (head_gate.shape == q.shape[:2] and head_gate.stride(1) == 1 and head_gate.dtype == q.dtype)
    T, H, d = q.shape
    G, dv = k_cache.shape[1], v_cache.shape[2]
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.shape[2] == d and v_cache.shape[1] == G
    assert out.shape == (T, H, dv) and q.stride(2) == 1 and out.stride(2) == 1 and q.dtype == out.dtype == k_cache.dtype == v_cache.dtype
    assert sink is None or (sink.dtype == torch.float32 and sink.numel() == H and sink.is_contiguous())
    assert req_to_token.dtype == torch.int32 and req_pool_indices.dtype == torch.int64 and positions.dtype == torch.int64
    assert tok_req is None or (tok_req.dtype == torch.int32 and tok_req.numel() == T)
    if blocks is not None:
        assert blocks.dtype == torch.int32 and blocks.dim() == 2 and blocks.shape[1] == 2 and blocks.is_contiguous()
        nb, num_splits = blocks.shape[0], 1
        assert max_run is not None, "runs come with their longest length"
    else:
        nb, max_run = T, 1
    scratch = torch.empty(num_splits * T * H * (dv + 2), dtype=torch.float32, device=q.device) if num_splits > 1 else None
    check(_lib_().mi355_window_attention_pooled(
        out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), _p(pooled_k) if pool > 0 else None,
        _p(pooled_v) if pool > 0 else None, req_to_token.data_ptr(), req_pool_indices.data_ptr(), _p(tok_req), positions.data_ptr(),
        _p(blocks), nb, _p(sink), _p(head_gate), head_gate.stride(0) if head_gate is not None else 0, q.stride(0), q.stride(1),
        out.stride(0), out.stride(1), req_to_token.stride(0), H, G, d, dv, int(window), int(pool), int(pool_div), float(scale),
        int(num_splits), _p(scratch), T, int(max_run), _dt(q), _stream(q)), "window_attention")
    return out


def pool_kv_blocks(k_cache: torch.Tensor, v_cache: torch.Tensor, pooled_k: torch.Tensor, pooled_v: torch.Tensor,
                   req_to_token: torch.Tensor, req_pool_indices: torch.Tensor, positions: torch.Tensor, pool: int, pool_div: int = 1,
                   tok_req=None) -> None:
    """For every token of the step whose position p ends a block of `pool` positions ((p + 1) % pool == 0): the mean of the
    block's cached keys (values) goes to pooled_k (pooled_v) [slot(p) // pool_div].  The step's keys and values must be in
    the caches already."""
    _gpu(k_cache, v_cache, pooled_k, pooled_v, req_to_token, req_pool_indices, positions, tok_req)
    G, d, dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[2]
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and pooled_k.is_contiguous() and pooled_v.is_contiguous()
    assert pooled_k.shape[1:] == (G, d) and pooled_v.shape[1:] == (G, dv) and pooled_k.dtype == pooled_v.dtype == k_cache.dtype == v_cache.dtype
    assert req_to_token.dtype == torch.int32 and req_pool_indices.dtype == torch.int64 and positions.dtype == torch.int64
    assert pool >= 1 and pool_div in (1, pool) and pooled_k.shape[0] * pool_div >= k_cache.shape[0]
    T = positions.numel()
    assert tok_req is None or (tok_req.dtype == torch.int32 and tok_req.numel() == T)
    check(_lib_().mi355_pool_kv_blocks(pooled_k.data_ptr(), pooled_v.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                       req_to_token.data_ptr(), req_pool_indices.data_ptr(), _p(tok_req), positions.data_ptr(), T,
                                       req_to_token.stride(0), G, d, dv, int(pool), int(pool_div), _dt(k_cache), _stream(k_cache)),
          "pool_kv_blocks")


def moe_route_scores(logits: torch.Tensor, correction: Optional[torch.Tensor], top: int, n_groups: int, keep_groups: int, scale: float,
                     score_fn: str = "sigmoid", group_best: int = 2, renorm: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
    """moe_route_grouped with its choices spelled out: scores "sigmoid" or "softmax" (over all experts), an optional
    selection-only correction, a group scoring the sum of its group_best (1 or 2) best members, weights renormalised or not."""
    _gpu(logits, correction)
    T, E = logits.shape
    assert logits.dtype == torch.float32 and logits.is_contiguous()
    assert correction is None or (correction.dtype == torch.float32 and correction.numel() == E)
    ids = torch.empty((T, top), dtype=torch.int32, device=logits.device)
    w = torch.empty((T, top), dtype=torch.float32, device=logits.device)
    check(_lib_().mi355_moe_route_scores(ids.data_ptr(), w.data_ptr(), logits.data_ptr(), _p(correction), T, E, int(top), int(n_groups),
                                         int(keep_groups), float(scale), {"sigmoid": 0, "softmax": 1}[score_fn], int(group_best),
                                         int(bool(renorm)), _stream(logits)), "moe_route_scores")
    return ids, w
