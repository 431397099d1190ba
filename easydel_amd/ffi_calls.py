"""JAX side of the ``jax.ffi`` shim: registers the handlers of ``csrc/rpa_ffi.cc`` and wraps each in a function with
the reference kernel's call signature.

This module needs ``jax`` (with a ROCm ``jaxlib``) and ``librpa_ffi.so`` (``easydel_amd.build.build_ffi()``); neither
exists in the image this repository is developed in, so the module is NOT compiled or run by the repository's tests
(they check that it parses and that its targets and the handlers of ``rpa_ffi.cc`` agree).  Nothing else in the
package imports it.  It is what a maintainer of the reference imports from the glue module that re-registers the
``ragged_page_attention_v2`` / ``_v3`` / ``unified_attention`` / ``multi_latent_ragged_page_attention`` operations
(the reference's call sites: ``easydel/operations/kernels/ragged_page_attention.py:281-313, 684-695, 732-746``,
``unified_attention.py:363-388``, ``multi_latent_ragged_page_attention.py:495-511``,
``easydel/caching/ragged_page/utils.py:302-387``).

Every wrapper sizes the scratch buffer from the static shapes (``rpa_attention_workspace_bytes``) and declares it as
an extra result, so XLA owns it; buffers updated in place are donated through ``input_output_aliases``.  The sizing
functions launch nothing, but they ask HIP for the current device's CU count and read the calling thread's test
knobs, so a size taken on the tracing thread may differ from what the executing thread and device would ask for.  That
is safe -- a call lays its workspace out from the bytes it is handed and splits less when they are fewer -- but a
different layout means a different split-K rounding, so results are only bit-identical for equal workspace sizes.
"""

from __future__ import annotations

import ctypes
from pathlib import Path

import jax
import jax.numpy as jnp
import numpy as np

_LIB_DIR = Path(__file__).resolve().parent / "lib"
TARGETS = ("RpaAttentionV2Ffi", "RpaAttentionV3Ffi", "RpaAttentionV3QuantisedFfi", "RpaUnifiedAttentionFfi",
           "RpaScatterSlicesFfi", "RpaScatterRaggedFfi", "RpaMlaAttentionFfi")

_abi = ctypes.CDLL(str(_LIB_DIR / "librpa_hip.so"))
_ffi = ctypes.CDLL(str(_LIB_DIR / "librpa_ffi.so"))
_abi.rpa_attention_workspace_bytes.restype = ctypes.c_size_t
_abi.rpa_attention_workspace_bytes.argtypes = [ctypes.c_int] * 9
_abi.rpa_mla_workspace_bytes.restype = ctypes.c_size_t
_abi.rpa_mla_workspace_bytes.argtypes = [ctypes.c_int] * 8
for _name in TARGETS:
    jax.ffi.register_ffi_target(_name, jax.ffi.pycapsule(getattr(_ffi, _name)), platform="ROCM")

_TAG = {jnp.dtype("float32"): 0, jnp.dtype("bfloat16"): 1, jnp.dtype("float8_e4m3fn"): 2, jnp.dtype("int8"): 3,
        jnp.dtype("float16"): 4}


def _stored_width(kv_pages, head_dim: int) -> int:
    """Elements of a stored head row: ``head_dim``, or its padded width (reference cache.py:640-647)."""
    stored = kv_pages.shape[-1]
    return 64 if (head_dim == 64 and stored == 128 and kv_pages.ndim == 5) else stored


def _workspace(T, S, M, page_size, Hq, Hkv, Dp, q_dtype, kv_dtype):
    n = _abi.rpa_attention_workspace_bytes(T, S, M, page_size, Hq, Hkv, Dp, _TAG[jnp.dtype(q_dtype)], _TAG[jnp.dtype(kv_dtype)])
    return jax.ShapeDtypeStruct((int(n),), jnp.uint8)


def _attrs(D, softmax_scale, sliding_window, logits_soft_cap, softmax_aux):
    return dict(softmax_scale=np.float32(D ** -0.5 if softmax_scale is None else softmax_scale),
                sliding_window=np.int32(sliding_window or 0), logits_soft_cap=np.float32(logits_soft_cap or 0.0),
                use_softmax_aux=np.bool_(softmax_aux is not None))


def _aux(softmax_aux, Hq):
    # one float32 logit per query head (ragged_page_attention.py:469-471); a dummy when there are no sinks
    return jnp.zeros((Hq,), jnp.float32) if softmax_aux is None else softmax_aux.astype(jnp.float32).reshape(Hq)


def attention_v2(query, kv_pages, context_lens, block_tables, query_start_loc, num_seqs, *, num_kv_heads,
                 softmax_scale=None, sliding_window=None, logits_soft_cap=None, softmax_aux=None):
    T, Hq, D = query.shape
    S, M = context_lens.shape[0], block_tables.size // context_lens.shape[0]
    ws = _workspace(T, S, M, kv_pages.shape[1], Hq, num_kv_heads, _stored_width(kv_pages, D), query.dtype, kv_pages.dtype)
    out, _ = jax.ffi.ffi_call("RpaAttentionV2Ffi", (jax.ShapeDtypeStruct(query.shape, query.dtype), ws))(
        query, kv_pages, context_lens, block_tables.reshape(-1), query_start_loc, num_seqs.reshape(-1), _aux(softmax_aux, Hq),
        num_kv_heads=np.int32(num_kv_heads), **_attrs(D, softmax_scale, sliding_window, logits_soft_cap, softmax_aux))
    return out


def attention_v3(query, key, value, kv_pages, context_lens, block_tables, query_start_loc, distribution, *,
                 softmax_scale=None, sliding_window=None, logits_soft_cap=None, softmax_aux=None):
    """Returns ``(out, kv_pages)``; ``key`` / ``value`` already in the cache dtype."""
    T, Hq, D = query.shape
    S, M = context_lens.shape[0], block_tables.size // context_lens.shape[0]
    ws = _workspace(T, S, M, kv_pages.shape[1], Hq, key.shape[1], _stored_width(kv_pages, D), query.dtype, kv_pages.dtype)
    out, pages, _ = jax.ffi.ffi_call(
        "RpaAttentionV3Ffi",
        (jax.ShapeDtypeStruct(query.shape, query.dtype), jax.ShapeDtypeStruct(kv_pages.shape, kv_pages.dtype), ws),
        input_output_aliases={3: 1},  # kv_pages operand -> kv_pages result: no copy of the pool per layer
    )(query, key, value, kv_pages, context_lens, block_tables.reshape(-1), query_start_loc, distribution, _aux(softmax_aux, Hq),
      **_attrs(D, softmax_scale, sliding_window, logits_soft_cap, softmax_aux))
    return out, pages


def attention_v3_quantised(query, key, value, kv_pages, kv_scales, context_lens, block_tables, query_start_loc, distribution, *,
                           softmax_scale=None, sliding_window=None, logits_soft_cap=None, softmax_aux=None):
    """Scaled fp8 / int8 pages: returns ``(out, kv_pages, kv_scales)``; ``key`` / ``value`` float32 or bfloat16."""
    T, Hq, D = query.shape
    S, M = context_lens.shape[0], block_tables.size // context_lens.shape[0]
    ws = _workspace(T, S, M, kv_pages.shape[1], Hq, key.shape[1], _stored_width(kv_pages, D), query.dtype, kv_pages.dtype)
    out, pages, scales, _ = jax.ffi.ffi_call(
        "RpaAttentionV3QuantisedFfi",
        (jax.ShapeDtypeStruct(query.shape, query.dtype), jax.ShapeDtypeStruct(kv_pages.shape, kv_pages.dtype),
         jax.ShapeDtypeStruct(kv_scales.shape, jnp.float32), ws),
        input_output_aliases={3: 1, 4: 2},
    )(query, key, value, kv_pages, kv_scales, context_lens, block_tables.reshape(-1), query_start_loc, distribution,
      _aux(softmax_aux, Hq), **_attrs(D, softmax_scale, sliding_window, logits_soft_cap, softmax_aux))
    return out, pages, scales


def unified_attention(query, key_cache, value_cache, context_lens, block_tables, query_start_loc, *, softmax_scale=None,
                      sliding_window=None, logits_soft_cap=None, softmax_aux=None):
    T, Hq, D = query.shape
    S, M = context_lens.shape[0], block_tables.size // context_lens.shape[0]
    ws = _workspace(T, S, M, key_cache.shape[1], Hq, key_cache.shape[2], D, query.dtype, key_cache.dtype)
    out, _ = jax.ffi.ffi_call("RpaUnifiedAttentionFfi", (jax.ShapeDtypeStruct(query.shape, query.dtype), ws))(
        query, key_cache, value_cache, context_lens, block_tables.reshape(-1), query_start_loc, _aux(softmax_aux, Hq),
        **_attrs(D, softmax_scale, sliding_window, logits_soft_cap, softmax_aux))
    return out


def kv_cache_update(new_kv_tokens, slice_indices, kv_cache_pages, total_update_slices, *, page_size=32, page_shard_index=0):
    """Drop-in for ``kv_cache_update_jax`` (same arguments); the pages are updated in place."""
    return jax.ffi.ffi_call("RpaScatterSlicesFfi", jax.ShapeDtypeStruct(kv_cache_pages.shape, kv_cache_pages.dtype),
                            input_output_aliases={2: 0})(
        new_kv_tokens.astype(kv_cache_pages.dtype), slice_indices, kv_cache_pages, total_update_slices.reshape(-1),
        page_size=np.int32(page_size), page_shard_index=np.int32(page_shard_index))


def page_scatter_ragged(key, value, kv_pages, context_lens, block_tables, query_start_loc, num_seqs):
    return jax.ffi.ffi_call("RpaScatterRaggedFfi", jax.ShapeDtypeStruct(kv_pages.shape, kv_pages.dtype),
                            input_output_aliases={2: 0})(
        key, value, kv_pages, context_lens, block_tables.reshape(-1), query_start_loc, num_seqs.reshape(-1))


def mla_attention(queries_nope, queries_pe, keys_values, keys_pe, kv_pages, context_lens, block_tables, query_start_loc,
                  distribution, *, softmax_scale, sliding_window=None, logits_soft_cap=None, softmax_aux=None):
    """Returns ``(out [T, Hq, kv_lora_rank], kv_pages)``; the caller passes ``(qk_nope_head_dim + qk_rope_head_dim) ** -0.5``."""
    T, Hq, rank = queries_nope.shape
    S, M = context_lens.shape[0], block_tables.size // context_lens.shape[0]
    page_size = kv_pages.shape[1] * kv_pages.shape[2] if kv_pages.ndim == 4 else kv_pages.shape[1]
    n = _abi.rpa_mla_workspace_bytes(T, S, M, page_size, Hq, rank, _TAG[jnp.dtype(queries_nope.dtype)], _TAG[jnp.dtype(kv_pages.dtype)])
    attrs = _attrs(rank, softmax_scale, sliding_window, logits_soft_cap, softmax_aux)
    out, pages, _ = jax.ffi.ffi_call(
        "RpaMlaAttentionFfi",
        (jax.ShapeDtypeStruct(queries_nope.shape, queries_nope.dtype), jax.ShapeDtypeStruct(kv_pages.shape, kv_pages.dtype),
         jax.ShapeDtypeStruct((int(n),), jnp.uint8)),
        input_output_aliases={4: 1},
    )(queries_nope, queries_pe, keys_values.astype(kv_pages.dtype), keys_pe.astype(kv_pages.dtype), kv_pages, context_lens,
      block_tables.reshape(-1), query_start_loc, distribution, _aux(softmax_aux, Hq), **attrs)
    return out, pages
