"""Tensor-level entry points: thin, checked wrappers over the C ABI.

PyTorch appears here only as the owner of device memory and streams (``data_ptr()`` and the
current HIP stream); all arithmetic happens in librpa_hip.so.  Every function raises if the
library is missing, if a tensor is not on a GPU, or if the C ABI reports an error.
"""

from __future__ import annotations

import math

import torch

from . import _lib

_DTYPE_TAG = {
    torch.float32: _lib.RPA_F32,
    torch.bfloat16: _lib.RPA_BF16,
    torch.float8_e4m3fn: _lib.RPA_FP8_E4M3,
    torch.int8: _lib.RPA_INT8,
    torch.float16: _lib.RPA_F16,
}

_workspaces: dict[tuple, torch.Tensor] = {}


def dtype_tag(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_TAG[dtype]
    except KeyError:
        raise NotImplementedError(f"dtype {dtype} is not supported by the ROCm ragged-page kernels") from None


def _dev(t: torch.Tensor, name: str) -> int:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor holding device memory, got {type(t).__name__}")
    if not t.is_cuda:
        raise RuntimeError(f"{name} is on {t.device}; the ROCm ragged-page kernels need GPU memory (no CPU fallback)")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    return t.data_ptr()


def _i32(t: torch.Tensor, name: str) -> int:
    if t.dtype != torch.int32:
        raise TypeError(f"{name} must be int32, got {t.dtype}")
    return _dev(t, name)


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def page_geometry(kv_pages: torch.Tensor, head_dim: int) -> tuple[int, int, int, int]:
    """(P, page_size, C, Dp) of a v2 ``[P, pg, 2*Hkv, D]`` or v3 ``[P, pg, groups, packing, Dp]`` page buffer.

    Both have token rows of ``C`` combined heads of ``Dp`` stored elements, K at even and V at odd
    combined heads.  The v3 shape for ``head_dim == 64`` packs K_h|V_h into one 128-wide row, which
    is the same bytes as rows of 64 (``Dp = 64``); any other head size is stored padded to a multiple
    of 128 (easydel/caching/ragged_page/cache.py:640-647), ``Dp > head_dim`` with zeros in the padding.
    """
    if kv_pages.ndim not in (4, 5):
        raise ValueError(f"kv_pages must be 4-D (v2) or 5-D (v3), got shape {tuple(kv_pages.shape)}")
    stored = kv_pages.shape[-1]
    if stored < head_dim:
        raise ValueError(f"kv_pages rows hold {stored} elements, fewer than head_dim {head_dim}")
    if head_dim == 64 and stored == 128 and kv_pages.ndim == 5:
        stored = 64  # K_h | V_h share one 128-wide row
    per_token = math.prod(kv_pages.shape[2:])
    return kv_pages.shape[0], kv_pages.shape[1], per_token // stored, stored


def workspace_bytes(T, S, M, page_size, Hq, Hkv, D, q_dtype: torch.dtype, kv_dtype: torch.dtype) -> int:
    return int(_lib.load().rpa_attention_workspace_bytes(T, S, M, page_size, Hq, Hkv, D, dtype_tag(q_dtype), dtype_tag(kv_dtype)))


def _workspace(device, nbytes: int) -> torch.Tensor:
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def page_scatter_slices(new_kv, slice_indices, num_slices, kv_cache_pages, *, page_size: int, page_shard_index: int = 0):
    """In-place v2 scatter: ``kv_cache_pages [N, C, D]`` (flat positions) <- ``new_kv [T, C, D]`` by slices."""
    lib = _lib.load()
    if new_kv.dtype != kv_cache_pages.dtype:
        raise TypeError(f"new_kv dtype {new_kv.dtype} != cache dtype {kv_cache_pages.dtype}")
    if slice_indices.ndim != 2 or slice_indices.shape[0] != 3:
        raise ValueError(f"slice_indices must be [3, N], got {tuple(slice_indices.shape)}")
    if tuple(new_kv.shape[1:]) != tuple(kv_cache_pages.shape[1:]):
        raise ValueError(f"token row shapes differ: {tuple(new_kv.shape[1:])} vs {tuple(kv_cache_pages.shape[1:])}")
    T, N, n_pos = new_kv.shape[0], slice_indices.shape[1], kv_cache_pages.shape[0]
    if T == 0 or N == 0 or n_pos == 0:
        return kv_cache_pages
    row_bytes = math.prod(new_kv.shape[1:]) * new_kv.element_size()
    _dev(kv_cache_pages, "kv_cache_pages")
    with torch.cuda.device(kv_cache_pages.device):  # the library queries and launches on HIP's current device
        _lib.check(lib.rpa_page_scatter_slices(
            _stream(kv_cache_pages), _dev(new_kv, "new_kv"), _i32(slice_indices, "slice_indices"),
            _i32(num_slices, "num_slices"), _dev(kv_cache_pages, "kv_cache_pages"), T, N, n_pos, int(page_size), row_bytes,
            int(page_shard_index)))
    return kv_cache_pages


def page_scatter_ragged(key, value, kv_pages, context_lens, block_tables, query_start_loc, num_seqs):
    """In-place v3 write: tokens of sequence i land at positions ``[ctx_i - q_len_i, ctx_i)`` of its pages."""
    lib = _lib.load()
    if key.dtype != kv_pages.dtype or value.dtype != kv_pages.dtype:
        raise TypeError(f"key/value dtype {key.dtype}/{value.dtype} must equal the cache dtype {kv_pages.dtype}")
    T, Hkv, D = key.shape
    P, pg, C, Dp = page_geometry(kv_pages, D)
    S = context_lens.shape[0]
    M = block_tables.numel() // S
    if T == 0:
        return kv_pages
    _dev(kv_pages, "kv_pages")
    with torch.cuda.device(kv_pages.device):  # the library queries and launches on HIP's current device
        _lib.check(lib.rpa_page_scatter_ragged(
            _stream(kv_pages), _dev(key, "key"), _dev(value, "value"), _dev(kv_pages, "kv_pages"),
            _i32(context_lens, "context_lens"), _i32(block_tables, "block_tables"), _i32(query_start_loc, "query_start_loc"),
            _i32(num_seqs, "num_seqs"), T, S, M, P, pg, Hkv, D, Dp, C, key.element_size()))
    return kv_pages


def page_scatter_ragged_quantised(key, value, kv_pages, kv_scales, context_lens, block_tables, query_start_loc, num_seqs):
    """In-place quantising v3 write into scaled fp8 / int8 pages: per (page, combined head) the scale only grows
    (``max(old, amax / qmax)``), tokens already in the page are re-coded when it does."""
    lib = _lib.load()
    if key.dtype != value.dtype or key.dtype not in (torch.float32, torch.bfloat16):
        raise TypeError(f"key/value must both be float32 or bfloat16, got {key.dtype}/{value.dtype}")
    if kv_pages.dtype not in (torch.float8_e4m3fn, torch.int8):
        raise TypeError(f"kv_pages must be float8_e4m3fn or int8 for the quantising write, got {kv_pages.dtype}")
    T, Hkv, D = key.shape
    P, pg, C, Dp = page_geometry(kv_pages, D)
    if kv_scales.dtype != torch.float32 or kv_scales.numel() != P * C:
        raise ValueError(f"kv_scales must be float32 [P={P}, C={C}]")
    S = context_lens.shape[0]
    M = block_tables.numel() // S
    if T == 0:
        return kv_pages, kv_scales
    _dev(kv_pages, "kv_pages")
    with torch.cuda.device(kv_pages.device):  # the library queries and launches on HIP's current device
        _lib.check(lib.rpa_page_scatter_ragged_quantised(
            _stream(kv_pages), _dev(key, "key"), _dev(value, "value"), _dev(kv_pages, "kv_pages"), _dev(kv_scales, "kv_scales"),
            _i32(context_lens, "context_lens"), _i32(block_tables, "block_tables"), _i32(query_start_loc, "query_start_loc"),
            _i32(num_seqs, "num_seqs"), T, S, M, P, pg, Hkv, D, Dp, C, dtype_tag(key.dtype), dtype_tag(kv_pages.dtype)))
    return kv_pages, kv_scales


def _sinks(softmax_aux, num_q_heads: int, device):
    """Attention-sink logits as the library takes them: float32 ``[Hq]`` on the query's device (the reference
    casts them to float32 and shards them by head, easydel/operations/kernels/ragged_page_attention.py:469-471).
    Returns ``(tensor kept alive by the caller, pointer)``; ``(None, None)`` without sinks."""
    if softmax_aux is None:
        return None, None
    if softmax_aux.ndim != 1 or softmax_aux.shape[0] != num_q_heads:
        raise NotImplementedError(f"softmax_aux must hold one sink logit per query head, shape [{num_q_heads}]; "
                                  f"got {tuple(softmax_aux.shape)}")
    if softmax_aux.device != device:
        raise ValueError(f"softmax_aux is on {softmax_aux.device}, the query on {device}")
    aux = softmax_aux.detach().to(torch.float32).contiguous()
    return aux, _dev(aux, "softmax_aux")


def _attn_common(query, kv_pages, context_lens, block_tables, num_kv_heads, softmax_scale, sliding_window, logits_soft_cap):
    T, Hq, D = query.shape
    P, pg, C, Dp = page_geometry(kv_pages, D)
    S = context_lens.shape[0]
    if block_tables.numel() % S:
        raise ValueError("block_tables size is not a multiple of the number of sequence rows")
    M = block_tables.numel() // S
    Hkv = int(num_kv_heads) if num_kv_heads is not None else C // 2
    scale = float(D) ** -0.5 if softmax_scale is None else float(softmax_scale)
    window = int(sliding_window) if sliding_window else 0
    cap = float(logits_soft_cap) if logits_soft_cap else 0.0
    return T, Hq, D, Dp, P, pg, C, S, M, Hkv, scale, window, cap


def ragged_paged_attention(query, kv_pages, context_lens, block_tables, query_start_loc, num_seqs, *,
                           softmax_scale=None, sliding_window=None, logits_soft_cap=None, kv_scales=None,
                           num_kv_heads=None, softmax_aux=None, out=None):
    """Read-only ragged paged attention; returns ``[T, Hq, D]`` in the query dtype."""
    lib = _lib.load()
    T, Hq, D, Dp, P, pg, C, S, M, Hkv, scale, window, cap = _attn_common(
        query, kv_pages, context_lens, block_tables, num_kv_heads, softmax_scale, sliding_window, logits_soft_cap)
    if out is None:
        out = torch.empty_like(query)
    if T == 0:
        return out
    qd, kd = dtype_tag(query.dtype), dtype_tag(kv_pages.dtype)
    for name, t in (("query", query), ("kv_pages", kv_pages), ("out", out)):
        _dev(t, name)
    aux, aux_ptr = _sinks(softmax_aux, Hq, query.device)
    ws = _workspace(query.device, int(lib.rpa_attention_workspace_bytes(T, S, M, pg, Hq, Hkv, Dp, qd, kd)))
    scales_ptr = None
    if kv_scales is not None:
        if kv_scales.dtype != torch.float32 or kv_scales.numel() != P * C:
            raise ValueError(f"kv_scales must be float32 [P={P}, C={C}]")
        scales_ptr = _dev(kv_scales, "kv_scales")
    with torch.cuda.device(query.device):  # the library queries and launches on HIP's current device
        _lib.check(lib.rpa_ragged_paged_attention(
            _stream(query), _dev(query, "query"), _dev(kv_pages, "kv_pages"), scales_ptr,
            _i32(context_lens, "context_lens"), _i32(block_tables, "block_tables"), _i32(query_start_loc, "query_start_loc"),
            _i32(num_seqs, "num_seqs"), _dev(out, "out"), ws.data_ptr(), ws.numel(),
            T, S, M, P, pg, Hq, Hkv, D, Dp, C, qd, kd, scale, window, cap, aux_ptr))
    return out


def unified_attention(query, key_cache, value_cache, context_lens, block_tables, query_start_loc, num_seqs=None, *,
                      softmax_scale=None, sliding_window=None, logits_soft_cap=None, kv_scales=None, softmax_aux=None,
                      out=None):
    """Ragged paged attention over separate K and V pools ``[P, page_size, Hkv, D]`` (the reference's
    unified-attention layout).  ``num_seqs`` is optional: without it every row of ``context_lens`` is live."""
    lib = _lib.load()
    if key_cache.shape != value_cache.shape or key_cache.dtype != value_cache.dtype:
        raise ValueError(f"key_cache {tuple(key_cache.shape)} {key_cache.dtype} and value_cache "
                         f"{tuple(value_cache.shape)} {value_cache.dtype} must match")
    if key_cache.ndim != 4:
        raise ValueError(f"key_cache must be [P, page_size, Hkv, D], got {tuple(key_cache.shape)}")
    T, Hq, D = query.shape
    P, pg, Hkv, Dk = key_cache.shape
    if Dk != D:
        raise NotImplementedError(f"cache head_dim {Dk} != query head_dim {D}")
    S = context_lens.shape[0]
    if block_tables.numel() % S:
        raise ValueError("block_tables size is not a multiple of the number of sequence rows")
    M = block_tables.numel() // S
    scale = float(D) ** -0.5 if softmax_scale is None else float(softmax_scale)
    window = int(sliding_window) if sliding_window else 0
    cap = float(logits_soft_cap) if logits_soft_cap else 0.0
    if out is None:
        out = torch.empty_like(query)
    if T == 0:
        return out
    qd, kd = dtype_tag(query.dtype), dtype_tag(key_cache.dtype)
    for name, t in (("query", query), ("key_cache", key_cache), ("value_cache", value_cache), ("out", out)):
        _dev(t, name)
    aux, aux_ptr = _sinks(softmax_aux, Hq, query.device)
    ws = _workspace(query.device, int(lib.rpa_attention_workspace_bytes(T, S, M, pg, Hq, Hkv, D, qd, kd)))
    scales_ptr = None
    if kv_scales is not None:
        if kv_scales.dtype != torch.float32 or kv_scales.numel() != P * 2 * Hkv:
            raise ValueError(f"kv_scales must be float32 [P={P}, 2*Hkv={2 * Hkv}]")
        scales_ptr = _dev(kv_scales, "kv_scales")
    with torch.cuda.device(query.device):  # the library queries and launches on HIP's current device
        _lib.check(lib.rpa_unified_attention(
            _stream(query), _dev(query, "query"), _dev(key_cache, "key_cache"), _dev(value_cache, "value_cache"), scales_ptr,
            _i32(context_lens, "context_lens"), _i32(block_tables, "block_tables"), _i32(query_start_loc, "query_start_loc"),
            None if num_seqs is None else _i32(num_seqs, "num_seqs"), _dev(out, "out"), ws.data_ptr(), ws.numel(),
            T, S, M, P, pg, Hq, Hkv, D, qd, kd, scale, window, cap, aux_ptr))
    return out


def ragged_paged_attention_v3(query, key, value, kv_pages, context_lens, block_tables, query_start_loc, distribution, *,
                              softmax_scale=None, sliding_window=None, logits_soft_cap=None, num_kv_heads=None,
                              softmax_aux=None, out=None):
    """Fused scatter + attention; updates ``kv_pages`` in place and returns ``(out, kv_pages)``."""
    lib = _lib.load()
    if key.dtype != kv_pages.dtype or value.dtype != kv_pages.dtype:
        raise TypeError(f"key/value dtype {key.dtype}/{value.dtype} must equal the cache dtype {kv_pages.dtype}")
    T, Hq, D, Dp, P, pg, C, S, M, Hkv, scale, window, cap = _attn_common(
        query, kv_pages, context_lens, block_tables, key.shape[1] if num_kv_heads is None else num_kv_heads,
        softmax_scale, sliding_window, logits_soft_cap)
    if out is None:
        out = torch.empty_like(query)
    if T == 0:
        return out, kv_pages
    qd, kd = dtype_tag(query.dtype), dtype_tag(kv_pages.dtype)
    for name, t in (("query", query), ("key", key), ("value", value), ("kv_pages", kv_pages), ("out", out)):
        _dev(t, name)
    aux, aux_ptr = _sinks(softmax_aux, Hq, query.device)
    ws = _workspace(query.device, int(lib.rpa_attention_workspace_bytes(T, S, M, pg, Hq, Hkv, Dp, qd, kd)))
    with torch.cuda.device(query.device):  # the library queries and launches on HIP's current device
        _lib.check(lib.rpa_ragged_paged_attention_v3(
            _stream(query), _dev(query, "query"), _dev(key, "key"), _dev(value, "value"), _dev(kv_pages, "kv_pages"),
            _i32(context_lens, "context_lens"), _i32(block_tables, "block_tables"), _i32(query_start_loc, "query_start_loc"),
            _i32(distribution, "distribution"), _dev(out, "out"), ws.data_ptr(), ws.numel(),
            T, S, M, P, pg, Hq, Hkv, D, Dp, C, qd, kd, scale, window, cap, aux_ptr))
    return out, kv_pages


def ragged_paged_attention_v3_static(query, key, value, kv_pages, context_lens, block_tables, query_start_loc, distribution, *,
                                     softmax_scale=None, sliding_window=None, logits_soft_cap=None, num_kv_heads=None,
                                     softmax_aux=None, out):
    """``ragged_paged_attention_v3`` through the entry point that allocates nothing: the caller passes ``out``, the
    scratch memory is the library's built-in per-GPU array (64 MiB; larger needs raise ``RpaError``).  Calls that
    overlap on one GPU share that array and race."""
    lib = _lib.load()
    if key.dtype != kv_pages.dtype or value.dtype != kv_pages.dtype:
        raise TypeError(f"key/value dtype {key.dtype}/{value.dtype} must equal the cache dtype {kv_pages.dtype}")
    T, Hq, D, Dp, P, pg, C, S, M, Hkv, scale, window, cap = _attn_common(
        query, kv_pages, context_lens, block_tables, key.shape[1] if num_kv_heads is None else num_kv_heads,
        softmax_scale, sliding_window, logits_soft_cap)
    if T == 0:
        return out, kv_pages
    qd, kd = dtype_tag(query.dtype), dtype_tag(kv_pages.dtype)
    aux_ptr = None
    if softmax_aux is not None:  # no conversion here: that would allocate
        if softmax_aux.dtype != torch.float32 or tuple(softmax_aux.shape) != (Hq,):
            raise ValueError(f"softmax_aux must be float32 [{Hq}] for the call that allocates nothing")
        aux_ptr = _dev(softmax_aux, "softmax_aux")
    with torch.cuda.device(query.device):  # the library queries and launches on HIP's current device
        _lib.check(lib.rpa_ragged_paged_attention_v3_static(
            _stream(query), _dev(query, "query"), _dev(key, "key"), _dev(value, "value"), _dev(kv_pages, "kv_pages"),
            _i32(context_lens, "context_lens"), _i32(block_tables, "block_tables"), _i32(query_start_loc, "query_start_loc"),
            _i32(distribution, "distribution"), _dev(out, "out"), T, S, M, P, pg, Hq, Hkv, D, Dp, C, qd, kd, scale, window, cap,
            aux_ptr))
    return out, kv_pages


def ragged_paged_attention_v3_quantised(query, key, value, kv_pages, kv_scales, context_lens, block_tables,
                                        query_start_loc, distribution, *, softmax_scale=None, sliding_window=None,
                                        logits_soft_cap=None, num_kv_heads=None, softmax_aux=None, out=None):
    """Fused quantising write + attention over scaled 8-bit pages; updates ``kv_pages`` and ``kv_scales`` in place
    and returns ``(out, kv_pages, kv_scales)``.  ``key`` / ``value`` are float32 or bfloat16."""
    lib = _lib.load()
    if key.dtype != value.dtype or key.dtype not in (torch.float32, torch.bfloat16):
        raise TypeError(f"key/value must both be float32 or bfloat16, got {key.dtype}/{value.dtype}")
    T, Hq, D, Dp, P, pg, C, S, M, Hkv, scale, window, cap = _attn_common(
        query, kv_pages, context_lens, block_tables, key.shape[1] if num_kv_heads is None else num_kv_heads,
        softmax_scale, sliding_window, logits_soft_cap)
    if kv_scales.dtype != torch.float32 or kv_scales.numel() != P * C:
        raise ValueError(f"kv_scales must be float32 [P={P}, C={C}]")
    if out is None:
        out = torch.empty_like(query)
    if T == 0:
        return out, kv_pages, kv_scales
    qd, kd = dtype_tag(query.dtype), dtype_tag(kv_pages.dtype)
    for name, t in (("query", query), ("key", key), ("value", value), ("kv_pages", kv_pages), ("kv_scales", kv_scales), ("out", out)):
        _dev(t, name)
    aux, aux_ptr = _sinks(softmax_aux, Hq, query.device)
    ws = _workspace(query.device, int(lib.rpa_attention_workspace_bytes(T, S, M, pg, Hq, Hkv, Dp, qd, kd)))
    with torch.cuda.device(query.device):  # the library queries and launches on HIP's current device
        _lib.check(lib.rpa_ragged_paged_attention_v3_quantised(
            _stream(query), _dev(query, "query"), _dev(key, "key"), _dev(value, "value"), _dev(kv_pages, "kv_pages"),
            _dev(kv_scales, "kv_scales"), _i32(context_lens, "context_lens"), _i32(block_tables, "block_tables"),
            _i32(query_start_loc, "query_start_loc"), _i32(distribution, "distribution"), _dev(out, "out"), ws.data_ptr(),
            ws.numel(), T, S, M, P, pg, Hq, Hkv, D, Dp, C, qd, dtype_tag(key.dtype), kd, scale, window, cap, aux_ptr))
    return out, kv_pages, kv_scales


def mla_row_geometry(kv_pages: torch.Tensor) -> tuple[int, int, int]:
    """(P, page_size, row_elems) of a latent page pool: ``[P, pg, row]`` or the reference's
    ``[P, pg / packing, packing, row]`` (easydel/caching/mla_ragged_page/cache.py:270-287), the same bytes."""
    if kv_pages.ndim == 3:
        return kv_pages.shape[0], kv_pages.shape[1], kv_pages.shape[2]
    if kv_pages.ndim == 4:
        return kv_pages.shape[0], kv_pages.shape[1] * kv_pages.shape[2], kv_pages.shape[3]
    raise ValueError(f"latent kv_pages must be 3-D or 4-D, got shape {tuple(kv_pages.shape)}")


def _mla_shapes(queries_nope, queries_pe, kv_pages, context_lens, block_tables):
    if queries_nope.ndim != 3 or queries_pe.ndim != 3 or queries_nope.shape[:2] != queries_pe.shape[:2]:
        raise ValueError("`queries_nope` and `queries_pe` must share [total_tokens, num_q_heads]. "
                         f"Got {tuple(queries_nope.shape)} vs {tuple(queries_pe.shape)}.")
    T, Hq, lkv = queries_nope.shape
    rope = queries_pe.shape[2]
    P, pg, row = mla_row_geometry(kv_pages)
    S = context_lens.shape[0]
    if block_tables.numel() % S:
        raise ValueError("block_tables size is not a multiple of the number of sequence rows")
    return T, Hq, lkv, rope, P, pg, row, S, block_tables.numel() // S


def mla_page_scatter(keys_values, keys_pe, kv_pages, context_lens, block_tables, query_start_loc, num_seqs):
    """In-place write of latent rows and rope keys: tokens of sequence i land at positions
    ``[ctx_i - q_len_i, ctx_i)`` of its pages (latent at 0, rope key at the padded latent width, padding zeroed)."""
    lib = _lib.load()
    if keys_values.dtype != kv_pages.dtype or keys_pe.dtype != kv_pages.dtype:
        raise TypeError(f"keys_values/keys_pe dtype {keys_values.dtype}/{keys_pe.dtype} must equal the cache dtype {kv_pages.dtype}")
    if keys_values.ndim != 2 or keys_pe.ndim != 2 or keys_values.shape[0] != keys_pe.shape[0]:
        raise ValueError(f"keys_values [T, kv_lora_rank] and keys_pe [T, rope] expected, got {tuple(keys_values.shape)}, {tuple(keys_pe.shape)}")
    T, lkv = keys_values.shape
    rope = keys_pe.shape[1]
    P, pg, row = mla_row_geometry(kv_pages)
    S = context_lens.shape[0]
    M = block_tables.numel() // S
    if T == 0:
        return kv_pages
    _dev(kv_pages, "kv_pages")
    with torch.cuda.device(kv_pages.device):  # the library queries and launches on HIP's current device
        _lib.check(lib.rpa_mla_page_scatter(
            _stream(kv_pages), _dev(keys_values, "keys_values"), _dev(keys_pe, "keys_pe"), _dev(kv_pages, "kv_pages"),
            _i32(context_lens, "context_lens"), _i32(block_tables, "block_tables"), _i32(query_start_loc, "query_start_loc"),
            _i32(num_seqs, "num_seqs"), T, S, M, P, pg, lkv, rope, row, keys_values.element_size()))
    return kv_pages


def mla_ragged_paged_attention(queries_nope, queries_pe, keys_values, keys_pe, kv_pages, context_lens, block_tables,
                               query_start_loc, distribution, *, softmax_scale=None, sliding_window=None,
                               logits_soft_cap=None, softmax_aux=None, out=None):
    """Multi-latent attention over latent pages, fused with the write of the new rows (``keys_values`` may be None:
    the pages are then read as they are).  Returns ``(out [T, Hq, kv_lora_rank], kv_pages)``."""
    lib = _lib.load()
    T, Hq, lkv, rope, P, pg, row, S, M = _mla_shapes(queries_nope, queries_pe, kv_pages, context_lens, block_tables)
    if queries_pe.dtype != queries_nope.dtype:
        raise TypeError(f"queries_pe dtype {queries_pe.dtype} != queries_nope dtype {queries_nope.dtype}")
    if keys_values is not None:
        if keys_pe is None:
            raise ValueError("multi_latent_ragged_page_attention requires `keys_pe`. Pass it as `keys_pe=` (or `k_pe=`).")
        if keys_values.dtype != kv_pages.dtype or keys_pe.dtype != kv_pages.dtype:
            raise TypeError(f"keys_values/keys_pe dtype {keys_values.dtype}/{keys_pe.dtype} must equal the cache dtype {kv_pages.dtype}")
        if tuple(keys_values.shape) != (T, lkv) or tuple(keys_pe.shape) != (T, rope):
            raise ValueError(f"keys_values {tuple(keys_values.shape)} / keys_pe {tuple(keys_pe.shape)} must be [{T}, {lkv}] / [{T}, {rope}]")
    if out is None:
        out = torch.empty_like(queries_nope)
    if T == 0:
        return out, kv_pages
    qd, kd = dtype_tag(queries_nope.dtype), dtype_tag(kv_pages.dtype)
    for name, t in (("queries_nope", queries_nope), ("queries_pe", queries_pe), ("kv_pages", kv_pages), ("out", out)):
        _dev(t, name)
    scale = float(lkv + rope) ** -0.5 if softmax_scale is None else float(softmax_scale)
    window = int(sliding_window) if sliding_window else 0
    cap = float(logits_soft_cap) if logits_soft_cap else 0.0
    aux, aux_ptr = _sinks(softmax_aux, Hq, queries_nope.device)
    ws = _workspace(queries_nope.device, int(lib.rpa_mla_workspace_bytes(T, S, M, pg, Hq, lkv, qd, kd)))
    with torch.cuda.device(queries_nope.device):  # the library queries and launches on HIP's current device
        _lib.check(lib.rpa_mla_ragged_paged_attention(
            _stream(queries_nope), _dev(queries_nope, "queries_nope"), _dev(queries_pe, "queries_pe"),
            None if keys_values is None else _dev(keys_values, "keys_values"),
            None if keys_values is None else _dev(keys_pe, "keys_pe"), _dev(kv_pages, "kv_pages"),
            _i32(context_lens, "context_lens"), _i32(block_tables, "block_tables"), _i32(query_start_loc, "query_start_loc"),
            _i32(distribution, "distribution"), _dev(out, "out"), ws.data_ptr(), ws.numel(),
            T, S, M, P, pg, Hq, lkv, rope, row, qd, kd, scale, window, cap, aux_ptr))
    return out, kv_pages
