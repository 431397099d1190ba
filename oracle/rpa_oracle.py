"""CPU oracle for the ragged-paged-attention path.  TEST INFRASTRUCTURE ONLY.

This module is the checker, never the product: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it.  Nothing under ``easydel_amd/`` imports it, and the product path
raises when its HIP library is missing instead of falling back to this code.

Everything here is a plain numpy (float64 / integer) restatement of what the
reference computes on this path.  Each function cites the reference lines it
follows.  The attention arithmetic itself lives in the third-party package
``ejkernel==0.0.78`` (pinned in the reference's ``pyproject.toml:36``), which is
not vendored under the reference tree and is not installed here; the attention
function below therefore restates the published ragged-paged-attention
algorithm as it is fixed by the reference's own call sites and in-tree
conventions (cited per line), and is pinned by closed forms, reductions to
textbook softmax attention (scipy), and invariants in ``tests/test_oracle_*``.

Pinning status
--------------
* ``kv_cache_update_ref`` / ``localize_slice_indices_ref``: pinned bit-exactly by
  the three vectors of ``tests/layers/caching/test_kv_cache_update_jax.py:84-180``.
* ``request_distribution_ref``: pinned by
  ``tests/inference/test_request_distribution_bounds.py:31-37`` and the host
  builder vectors ``:47-117``.
* ``storage_layout_ref``: pinned by
  ``tests/layers/caching/test_ragged_page_dtype_compat.py:34-60`` (packing/groups).
* ``slot_mapping_v2_ref``: pinned by closed form (each scheduled token appears
  once, ``dst = page_table[r, t // pg] * pg + t % pg``) and a round trip through
  the scatter.
* ``ragged_paged_attention_ref``: the reference holds no golden vector for the
  attention output (its only test of the call mocks the kernel out); pinned by
  mathematics only -- see ``tests/test_oracle_attention.py`` -- and therefore
  "parity unpinned" against ejkernel.  The residual conventions that only an
  import of ejkernel could confirm (where its XLA path rounds to bf16, what it
  writes to padded rows, the mask value of fully masked rows) are covered by
  comparing valid rows only, at the stated tolerances.  Its ``softmax_aux`` (attention sinks) arm is
  likewise unpinned against ejkernel; it is pinned to the published GPT-OSS attention (the
  ``transformers`` library's eager implementation, run on dense inputs) and to the closed form
  ``out = out_without_sink * sigmoid(logsumexp(scores) - sink)``.
* ``page_scatter_ragged_ref`` (the fused v3 write): no reference vector exists
  (it runs inside ejkernel); pinned by equivalence with the v2 scatter driven by
  ``slot_mapping_v2_ref`` on the same batch.
* e4m3fn / bf16 codecs: pinned against ``torch``'s CPU casts over all codes.
* ``page_scatter_ragged_quantised_ref``: the scaled 8-bit page format has no counterpart in
  the reference (its ragged pages carry no scales); this function defines it.  Pinned by
  invariants in ``tests/test_oracle_formats.py`` (round-trip error bounds, monotone scales,
  equivalence with one-shot quantisation when nothing is re-coded, placement equal to the
  unquantised ragged write).
* ``mla_ragged_paged_attention_ref`` / ``mla_page_scatter_ref``: the arithmetic lives in ejkernel and the
  reference holds no vector for it: "parity unpinned" against ejkernel.  Pinned in ``tests/test_oracle_mla.py`` to the
  reference's own non-absorbed branch of the same layer (keys and values decompressed through the up-projection,
  then ordinary attention, ``layers/attention/_unified.py:1240-1248, 1380-1395``), i.e. to
  ``ragged_paged_attention_ref`` on decompressed pages, and to the reductions of that function's tests.
  ``mla_page_layout_ref`` is pinned by the shape arithmetic of ``caching/mla_ragged_page/cache.py:198-201``.
* ``dp_local_shard_ref`` (one data-parallel rank's view of the metadata when pages are sharded over ranks): no
  reference vector exists; pinned in ``tests/test_oracle_dp_local.py`` by what the scheme must guarantee -- every
  scheduled token is owned by exactly one rank, a page id owned by the rank maps to itself minus the rank's first page
  and any other id is clipped into the local pool, and the float32 sum over ranks of the ranks' masked attention
  outputs equals the attention over the whole pool when every sequence's pages live on the rank of its row.
"""

from __future__ import annotations

import math

import numpy as np

# --------------------------------------------------------------------------------------
# Number formats (numpy bit arithmetic; no ml_dtypes in this image)
# --------------------------------------------------------------------------------------


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round float32 to bfloat16 (round-to-nearest-even), returned as uint16 bit patterns."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounded = u >> np.uint32(16)  # (u + 0x7FFF + lsb of the kept half) >> 16, in place: the test pools are 10^8 elements
    rounded &= np.uint32(1)
    rounded += np.uint32(0x7FFF)
    rounded += u
    rounded >>= np.uint32(16)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    if nan.any():
        rounded[nan] = (u[nan] >> np.uint32(16)) | np.uint32(0x0040)
    return rounded.astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    """Widen bfloat16 bit patterns (uint16) to float32 exactly."""
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def e4m3fn_decode_table() -> np.ndarray:
    """All 256 OCP float8 e4m3fn codes as float32 (1-4-3, bias 7, no inf, 0x7f/0xff NaN)."""
    out = np.empty(256, dtype=np.float32)
    for c in range(256):
        s, e, m = c >> 7, (c >> 3) & 15, c & 7
        if e == 15 and m == 7:
            v = float("nan")
        elif e == 0:
            v = math.ldexp(m / 8.0, -6)
        else:
            v = math.ldexp(1.0 + m / 8.0, e - 7)
        out[c] = -v if s else v
    return out


_E4M3_TABLE = e4m3fn_decode_table()


def e4m3fn_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return _E4M3_TABLE[np.ascontiguousarray(b, dtype=np.uint8)]


def f32_to_e4m3fn_bits(x: np.ndarray) -> np.ndarray:
    """Round float32 to e4m3fn codes, nearest-even, saturating at +-448."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    pos = _E4M3_TABLE[:127].astype(np.float64)  # codes 0..126 ascending, 126 -> 448
    a = np.minimum(np.abs(x.astype(np.float64)), 448.0)
    hi = np.searchsorted(pos, a, side="left").clip(0, 126)
    lo = np.maximum(hi - 1, 0)
    dlo, dhi = a - pos[lo], pos[hi] - a
    pick_hi = (dhi < dlo) | ((dhi == dlo) & ((hi & 1) == 0))
    code = np.where(pick_hi, hi, lo).astype(np.uint8)
    code = np.where(np.isnan(x), np.uint8(0x7F), code)
    return (code | (np.signbit(x).astype(np.uint8) << 7)).astype(np.uint8)


# dtype tags shared with the C ABI (include/rpa_hip.h: rpa_dtype)
def cast_e4m3fn_ref(x: np.ndarray) -> np.ndarray:
    """The plain cast to e4m3fn codes the reference applies to K/V headed for an fp8 cache
    (``key.astype(kv_cache_dtype)``, operations/kernels/ragged_page_attention.py:570-580): round to nearest
    even, and -- the format has no infinity -- whatever rounds beyond +-448 (|x| > 464; the tie at 464 goes to the
    even code, 448) becomes NaN; nothing saturates.  jax's cast runs in ml_dtypes / XLA, neither present here: "parity unpinned" against them; pinned
    against torch's CPU cast (same documented rule) in tests/test_oracle_formats.py."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    code = f32_to_e4m3fn_bits(x)
    over = np.abs(x.astype(np.float64)) > 464.0  # 464 is halfway between 448 and the (absent) 480
    return np.where(over, code | np.uint8(0x7F), code).astype(np.uint8)


F32, BF16, FP8_E4M3, INT8, F16 = 0, 1, 2, 3, 4


def decode_array(raw: np.ndarray, dtype_tag: int) -> np.ndarray:
    """Storage bits -> float64 values for the four element formats of the path."""
    if dtype_tag == F32:
        return np.asarray(raw, dtype=np.float32).astype(np.float64)
    if dtype_tag == BF16:
        return bf16_bits_to_f32(raw).astype(np.float64)
    if dtype_tag == FP8_E4M3:
        return e4m3fn_bits_to_f32(raw).astype(np.float64)
    if dtype_tag == INT8:
        return np.asarray(raw, dtype=np.int8).astype(np.float64)
    if dtype_tag == F16:
        return np.asarray(raw, dtype=np.float16).astype(np.float64)
    raise ValueError(f"unknown dtype tag {dtype_tag}")


# --------------------------------------------------------------------------------------
# Integer metadata
# --------------------------------------------------------------------------------------


def request_distribution_ref(scheduled, context_lens) -> np.ndarray:
    """[decode_end, prefill_end, total] -- easydel/operations/kernels/ragged_page_attention.py:177-187."""
    scheduled = np.asarray(scheduled, dtype=np.int32)
    context_lens = np.asarray(context_lens, dtype=np.int32)
    has = scheduled > 0
    dec = (scheduled == 1) & (context_lens > 1) & has
    n_dec = int(dec.sum())
    return np.array([n_dec, n_dec + int((has & ~dec).sum()), int(has.sum())], dtype=np.int32)


def dp_local_shard_ref(shard_index: int, num_shards: int, context_lens, pages_tables, query_start_loc, local_num_pages: int,
                       total_tokens: int) -> dict:
    """One data-parallel rank's metadata when the page pool is sharded over ranks --
    easydel/operations/kernels/ragged_page_attention.py:645-712 (the body of the shard_map before the sum over ranks).
    The rank takes rows ``[shard * S/n, (shard + 1) * S/n)`` of the lengths and page tables and the matching
    ``S/n + 1`` entries of ``query_start_loc`` (:650-672; token indices stay global), recomputes the request distribution
    (:674-676), rebases page ids by ``shard * local_num_pages`` and clips them to ``[0, local_num_pages - 1]`` (:678-681),
    and keeps the output rows of its own live requests only (:699-712: ``token_mask``)."""
    context_lens = np.asarray(context_lens, dtype=np.int32)
    S = context_lens.shape[0]
    if S % num_shards:
        raise ValueError("metadata rows do not divide over the shards")
    rows = S // num_shards
    r0 = shard_index * rows
    local_ctx = context_lens[r0:r0 + rows].copy()
    local_tables = np.asarray(pages_tables, dtype=np.int32).reshape(S, -1)[r0:r0 + rows]
    local_qsl = np.asarray(query_start_loc, dtype=np.int32)[r0:r0 + rows + 1].copy()
    dist = request_distribution_ref(local_qsl[1:] - local_qsl[:-1], local_ctx)
    rebased = np.clip(local_tables - np.int32(shard_index * local_num_pages), 0, local_num_pages - 1).astype(np.int32)
    mask = np.zeros(total_tokens, dtype=bool)
    for r in range(rows):
        if r < int(dist[2]):
            mask[local_qsl[r]:local_qsl[r + 1]] = True
    return dict(context_lens=local_ctx, block_tables=rebased.reshape(-1), query_start_loc=local_qsl, distribution=dist,
                token_mask=mask)


def storage_layout_ref(num_kv_heads: int, head_dim: int, bits: int) -> dict:
    """v3 page storage geometry -- easydel/caching/ragged_page/cache.py:143-158, 616-647, 695-729."""
    if 32 % bits:
        raise ValueError("bit width must divide 32")
    packing = 32 // bits
    base = num_kv_heads if head_dim == 64 else 2 * num_kv_heads
    combined = -(-base // packing) * packing
    dp = 128 if head_dim == 64 else -(-head_dim // 128) * 128
    return {"packing": packing, "combined": combined, "groups": combined // packing, "head_dim": dp}


def slot_mapping_v2_ref(scheduled, num_computed, page_table, page_size: int, slices_per_page: int = 1):
    """Per-(request, page) copy slices -- easydel/caching/_metadatabuilder.py:783-882.

    Written as the obvious double loop (the reference vectorises it); returns
    ``(slot_mapping[3, padded], total_slices)``.
    """
    scheduled = np.asarray(scheduled, dtype=np.int64)
    num_computed = np.asarray(num_computed, dtype=np.int64)
    cols, src = [], 0
    for r in range(len(scheduled)):
        n = int(scheduled[r])
        if n <= 0:
            continue
        start, end = int(num_computed[r]), int(num_computed[r]) + n
        for page_idx in range(start // page_size, (end - 1) // page_size + 1):
            lo = max(start, page_idx * page_size)
            hi = min(end, (page_idx + 1) * page_size)
            cols.append((int(page_table[r, page_idx]) * page_size + lo % page_size, src, hi - lo))
            src += hi - lo
    total = len(cols)
    padded = max(-(-total // slices_per_page) * slices_per_page, 1)
    out = np.zeros((3, padded), dtype=np.int32)
    if total:
        out[:, :total] = np.asarray(cols, dtype=np.int32).T
    return out, total


# --------------------------------------------------------------------------------------
# Page scatter
# --------------------------------------------------------------------------------------


def localize_slice_indices_ref(slice_indices, total_update_slices, *, page_size, local_flat_cache_positions,
                               page_shard_index=0) -> np.ndarray:
    """easydel/caching/ragged_page/utils.py:66-123."""
    si = np.asarray(slice_indices)
    n_valid = int(np.asarray(total_update_slices).reshape(-1)[0])
    n = si.shape[1]
    if n == 0:
        return si
    local_pages = max(int(local_flat_cache_positions) // int(page_size), 1)
    out = np.zeros_like(si)
    for c in range(n):
        dst = int(si[0, c])
        page, off = dst // page_size, dst % page_size  # floor semantics, as jnp // and %
        local_page = page - int(page_shard_index) * local_pages
        if c < n_valid and 0 <= local_page < local_pages:
            out[0, c] = local_page * page_size + off
            out[1, c] = si[1, c]
            out[2, c] = si[2, c]
    return out


def kv_cache_update_ref(new_kv_tokens, slice_indices, kv_cache_pages, total_update_slices, *, page_size=32,
                        page_shard_index=0) -> np.ndarray:
    """The v2 page scatter -- easydel/caching/ragged_page/utils.py:302-387.

    ``new_kv_tokens [T, C, D]``, ``kv_cache_pages [N, C, D]`` (flat cache positions).  Bit copy of
    whole token rows; element type is opaque.  Follows the reference's packed-token expansion:
    packed token ``t`` belongs to the first slice whose cumulative end exceeds ``t``; tokens past
    the packed total, or whose source row is out of range, are dropped; a destination outside
    ``[0, N)`` is dropped (``mode="drop"``), negative destinations wrap once as numpy/jnp indexing does.
    """
    new_kv = np.asarray(new_kv_tokens)
    pages = np.array(kv_cache_pages, copy=True)
    si = localize_slice_indices_ref(slice_indices, total_update_slices, page_size=page_size,
                                    local_flat_cache_positions=pages.shape[0], page_shard_index=page_shard_index)
    if pages.size == 0:
        return pages
    n_valid = int(np.asarray(total_update_slices).reshape(-1)[0])
    n_tok, n_pos = new_kv.shape[0], pages.shape[0]
    packed = 0
    for c in range(si.shape[1]):
        ln = int(si[2, c]) if c < n_valid else 0
        for off in range(max(ln, 0)):
            if packed >= n_tok:
                break
            src, dst = int(si[1, c]) + off, int(si[0, c]) + off
            packed += 1
            if not (0 <= src < n_tok):
                continue
            if dst < 0:
                dst += n_pos
            if 0 <= dst < n_pos:
                pages[dst] = new_kv[src]
    return pages


def page_scatter_ragged_ref(key, value, kv_pages, context_lens, block_tables, query_start_loc, num_seqs) -> np.ndarray:
    """The write half of the fused v3 op (call site ragged_page_attention.py:732-746).

    Sequence ``i`` writes ``key/value[qsl[i]:qsl[i+1]]`` to token positions ``[ctx_i - q_len_i, ctx_i)`` of
    its pages; K of head ``h`` goes to combined head ``2h``, V to ``2h+1`` (cache.py:928, 954-973).
    ``kv_pages [P, pg, C, D]`` with ``C >= 2*Hkv``; ``block_tables [S, M]``.
    """
    pages = np.array(kv_pages, copy=True)
    pg = pages.shape[1]
    hkv = key.shape[1]
    bt = np.asarray(block_tables).reshape(len(context_lens), -1)
    for i in range(int(np.asarray(num_seqs).reshape(-1)[0])):
        q0, q1 = int(query_start_loc[i]), int(query_start_loc[i + 1])
        ctx = int(context_lens[i])
        for r in range(q1 - q0):
            pos = ctx - (q1 - q0) + r
            if pos < 0:
                continue
            page = int(bt[i, pos // pg])
            pages[page, pos % pg, 0:2 * hkv:2] = key[q0 + r]
            pages[page, pos % pg, 1:2 * hkv:2] = value[q0 + r]
    return pages


QMAX = {FP8_E4M3: 448.0, INT8: 127.0}


def quantise_codes(y: np.ndarray, kv_dtype: int) -> np.ndarray:
    """Scaled values -> 8-bit codes as raw uint8: clamp to the code range, round to nearest even."""
    y = np.ascontiguousarray(y, dtype=np.float32)
    q = np.float32(QMAX[kv_dtype])
    y = np.minimum(np.maximum(y, -q), q)
    if kv_dtype == FP8_E4M3:
        return f32_to_e4m3fn_bits(y)
    return np.rint(y).astype(np.int8).view(np.uint8)


def decode_codes(raw: np.ndarray, kv_dtype: int) -> np.ndarray:
    raw = np.ascontiguousarray(raw).view(np.uint8)
    if kv_dtype == FP8_E4M3:
        return e4m3fn_bits_to_f32(raw)
    return raw.view(np.int8).astype(np.float32)


def page_scatter_ragged_quantised_ref(key, value, kv_codes, kv_scales, context_lens, block_tables, query_start_loc,
                                      num_seqs, *, kv_dtype: int):
    """Quantising form of the ragged page write.  The scaled 8-bit page format belongs to this build (the
    reference's ragged pages have no scales), so this function defines it; the kernel must match it bit for bit.

    ``key/value [T, Hkv, D]`` float32 values; ``kv_codes [P, pg, C, D]`` raw uint8 codes; ``kv_scales [P, C]``
    float32; value = code * scale[page, combined head].  Per (sequence, page it writes to, combined head), with
    all arithmetic in float32:
      * the new tokens of the page are ``[first, first + n)`` (token offsets inside the page);
      * ``old = 0`` if ``first == 0`` (the page starts here: whatever scale it held belonged to an earlier owner),
        else the stored scale;
      * ``new = max(old, amax(|new values|) / qmax)``, and 1.0 if that is 0;
      * if ``new > old`` and ``first > 0`` the tokens already in the page are re-coded:
        ``code <- quant((decode(code) * old) / new)``;
      * the new tokens are coded ``quant(x / new)``, and ``new`` is stored.
    ``quant`` clamps to the code range and rounds to nearest even (``quantise_codes``).
    Returns ``(codes, scales)``.
    """
    codes = np.array(kv_codes, copy=True).view(np.uint8)
    scales = np.array(kv_scales, dtype=np.float32, copy=True)
    pg = codes.shape[1]
    hkv = key.shape[1]
    qmax = np.float32(QMAX[kv_dtype])
    bt = np.asarray(block_tables).reshape(len(context_lens), -1)
    key = np.ascontiguousarray(key, dtype=np.float32)
    value = np.ascontiguousarray(value, dtype=np.float32)
    for i in range(int(np.asarray(num_seqs).reshape(-1)[0])):
        q0, q1 = int(query_start_loc[i]), int(query_start_loc[i + 1])
        ctx = int(context_lens[i])
        q_len = q1 - q0
        pos = max(ctx - q_len, 0)
        while pos < ctx:
            j, first = pos // pg, pos % pg
            n = min(ctx, (j + 1) * pg) - pos
            page = int(bt[i, j])
            t0 = q0 + (pos - (ctx - q_len))
            for c in range(2 * hkv):
                src = (value if c & 1 else key)[t0:t0 + n, c >> 1]  # [n, D]
                old = np.float32(0.0) if first == 0 else scales[page, c]
                new = np.maximum(old, np.float32(np.abs(src).max()) / qmax).astype(np.float32)
                if new == 0:
                    new = np.float32(1.0)
                if new > old and first > 0:
                    prev = decode_codes(codes[page, :first, c], kv_dtype)
                    codes[page, :first, c] = quantise_codes((prev * old) / new, kv_dtype)
                codes[page, first:first + n, c] = quantise_codes(src / new, kv_dtype)
                scales[page, c] = new
            pos += n
    return codes, scales


# --------------------------------------------------------------------------------------
# Attention
# --------------------------------------------------------------------------------------


def ragged_paged_attention_ref(query, kv_pages, context_lens, block_tables, query_start_loc, num_seqs, *,
                               softmax_scale=None, sliding_window=None, logits_soft_cap=None, kv_scales=None,
                               num_kv_heads=None, softmax_aux=None) -> np.ndarray:
    """Ragged paged attention in float64 (operation called at ragged_page_attention.py:281-313 / 732-746).

    ``query [T, Hq, D]`` and ``kv_pages [P, pg, C, D]`` are *decoded values* (float arrays).  Conventions, each
    fixed in-tree by the reference:
      * K of KV head ``h`` is combined head ``2h``, V is ``2h+1``                      (cache.py:954-973)
      * query row ``r`` of sequence ``i`` sits at position ``ctx_i - q_len_i + r``      (batch_preparer.py:645-657)
      * GQA: query head ``h`` reads KV head ``h // (Hq/Hkv)``                          (_operation_impl.py:264-267)
      * scores are scaled, then optionally soft-capped ``cap*tanh(s/cap)``, then masked;
        key ``j`` is visible iff ``j <= pos`` and, with window ``W``, ``j > pos - W``
        (``W`` keys including self; single_type_cache_manager.py:497)
      * ``softmax_scale=None`` means ``D**-0.5``                                       (ragged_page_attention.py:784)
      * ``kv_scales [P, C]`` (this build's quantised-page format): value = code * scale[page, combined head].
      * ``softmax_aux [Hq]``: attention sinks, one logit per query head, float32
        (ragged_page_attention.py:469-471, fed by modules/gpt_oss/modeling_gpt_oss.py:436-442).  The sink
        arithmetic lives in ejkernel; restated here is the published GPT-OSS definition that parameter belongs
        to: the softmax runs over ``[scores, sink]`` and the sink's column is dropped, so the sink enters the
        denominator only, as is (no scale, no soft cap, never masked).
    Rows of padded tokens (``t >= qsl[num_seqs]``) and of sequences with ``q_len == 0`` are returned as zeros.
    """
    q = np.asarray(query, dtype=np.float64)
    pages = np.asarray(kv_pages, dtype=np.float64)
    n_tok, hq, d = q.shape
    pg = pages.shape[1]
    hkv = int(num_kv_heads) if num_kv_heads is not None else pages.shape[2] // 2
    group = hq // hkv
    scale = float(d) ** -0.5 if softmax_scale is None else float(softmax_scale)
    bt = np.asarray(block_tables).reshape(len(context_lens), -1)
    out = np.zeros((n_tok, hq, d), dtype=np.float64)
    sinks = None
    if softmax_aux is not None:
        sinks = np.asarray(softmax_aux, dtype=np.float64).reshape(-1)
        if sinks.shape[0] != hq:
            raise ValueError(f"softmax_aux must hold one logit per query head ({hq}), got {sinks.shape[0]}")
    for i in range(int(np.asarray(num_seqs).reshape(-1)[0])):
        q0, q1 = int(query_start_loc[i]), int(query_start_loc[i + 1])
        ctx, q_len = int(context_lens[i]), q1 - q0
        if q_len <= 0 or ctx <= 0:
            continue
        n_pages = -(-ctx // pg)
        ids = bt[i, :n_pages]
        seq = pages[ids]  # [n_pages, pg, C, D]
        if kv_scales is not None:
            seq = seq * np.asarray(kv_scales, dtype=np.float64)[ids][:, None, :, None]
        seq = seq.reshape(n_pages * pg, pages.shape[2], d)[:ctx]
        pos = ctx - q_len + np.arange(q_len)
        j = np.arange(ctx)
        visible = j[None, :] <= pos[:, None]
        if sliding_window is not None and int(sliding_window) > 0:
            visible &= j[None, :] > (pos[:, None] - int(sliding_window))
        for h in range(hq):
            k = seq[:, 2 * (h // group), :]
            v = seq[:, 2 * (h // group) + 1, :]
            s = (q[q0:q1, h, :] @ k.T) * scale
            if logits_soft_cap is not None and float(logits_soft_cap) > 0:
                s = float(logits_soft_cap) * np.tanh(s / float(logits_soft_cap))
            s = np.where(visible, s, -np.inf)
            m = s.max(axis=1, keepdims=True)
            if sinks is not None:
                m = np.maximum(m, sinks[h])
            m = np.where(np.isfinite(m), m, 0.0)
            p = np.exp(s - m)
            denom = p.sum(axis=1, keepdims=True)
            if sinks is not None:
                denom = denom + np.exp(sinks[h] - m)
            out[q0:q1, h, :] = (p @ v) / np.where(denom > 0, denom, 1.0)
    return out


# --------------------------------------------------------------------------------------
# Multi-latent attention (MLA) over latent ragged pages
# --------------------------------------------------------------------------------------
def mla_page_layout_ref(kv_lora_rank: int, qk_rope_head_dim: int, page_size: int, bits: int = 16) -> dict:
    """Shape of the latent page pool (caching/mla_ragged_page/cache.py:198-201, 250-287).

    One row per token, no head axis: the latent ``kv_lora_rank`` values and the rope key ``qk_rope_head_dim`` values,
    each padded to a multiple of 128 on its own (``:257-258``); tokens are packed ``32 // bits`` to a storage row
    (``:199-200``), which in memory is the same as ``[P, page_size', row]`` with ``page_size'`` rounded up to the packing.
    The rope part is taken to start at the padded latent width (the reference states only the total; where ejkernel
    puts the parts inside a row cannot be read from the tree, and for ``kv_lora_rank`` a multiple of 128 -- every model
    that uses the operation has 512 -- the two readings coincide).
    """
    packing = 32 // int(bits)
    lkv_pad = -(-int(kv_lora_rank) // 128) * 128
    rope_pad = -(-int(qk_rope_head_dim) // 128) * 128
    per = -(-int(page_size) // packing)
    return dict(kv_packing=packing, page_size_per_kv_packing=per, kv_dim_padded=lkv_pad + rope_pad, rope_offset=lkv_pad,
                shape_tail=(per, packing, lkv_pad + rope_pad))


def mla_page_scatter_ref(keys_values, keys_pe, kv_pages, context_lens, block_tables, query_start_loc, num_seqs) -> np.ndarray:
    """The write half of the MLA operation (call site multi_latent_ragged_page_attention.py:495-511, 611-624).

    ``kv_pages [P, pg, row]``; sequence ``i`` writes the latent rows ``keys_values[qsl[i]:qsl[i+1]]`` and the rope keys
    ``keys_pe[...]`` to token positions ``[ctx_i - q_len_i, ctx_i)`` of its pages (the positions of the fused v3 write,
    the operation takes the same metadata): latent at ``[0, lkv)``, rope key at ``[rope_offset, rope_offset + rope)``,
    the padding of a written row set to zero.
    """
    pages = np.array(kv_pages, copy=True)
    pg, row = pages.shape[1], pages.shape[2]
    lkv, rope = keys_values.shape[1], keys_pe.shape[1]
    off = -(-lkv // 128) * 128
    assert off + rope <= row
    bt = np.asarray(block_tables).reshape(len(context_lens), -1)
    for i in range(int(np.asarray(num_seqs).reshape(-1)[0])):
        q0, q1 = int(query_start_loc[i]), int(query_start_loc[i + 1])
        ctx = int(context_lens[i])
        for r in range(q1 - q0):
            pos = ctx - (q1 - q0) + r
            if pos < 0:
                continue
            page = int(bt[i, pos // pg])
            pages[page, pos % pg, :] = 0
            pages[page, pos % pg, :lkv] = keys_values[q0 + r]
            pages[page, pos % pg, off:off + rope] = keys_pe[q0 + r]
    return pages


def mla_ragged_paged_attention_ref(queries_nope, queries_pe, kv_pages, context_lens, block_tables, query_start_loc,
                                   num_seqs, *, kv_lora_rank, qk_rope_head_dim, softmax_scale=None, sliding_window=None,
                                   logits_soft_cap=None, softmax_aux=None) -> np.ndarray:
    """Multi-latent attention over latent pages in float64 (operation called at
    multi_latent_ragged_page_attention.py:495-511; inputs and output as its caller builds and consumes them,
    layers/attention/_unified.py:1280-1375).

    ``queries_nope [T, Hq, lkv]`` are the queries already multiplied by the key half of the up-projection ("weight
    absorption", ``_unified.py:1292-1298``), ``queries_pe [T, Hq, rope]`` their rotary part; every head reads the same
    row per token: score = ``scale * (q_nope . latent + q_pe . k_pe)``, the values are the latent rows themselves, and the
    output ``[T, Hq, lkv]`` is the softmax-weighted sum of latent rows, which the caller multiplies by the value half
    of the up-projection (``:1366-1371``).  Masking, window, soft cap, sinks, positions and padding as in
    ``ragged_paged_attention_ref``.  ``softmax_scale=None`` means ``(lkv + rope) ** -0.5`` here; the caller always
    passes ``(qk_nope_head_dim + qk_rope_head_dim) ** -0.5`` (``:1310``).
    """
    qn = np.asarray(queries_nope, dtype=np.float64)
    qp = np.asarray(queries_pe, dtype=np.float64)
    pages = np.asarray(kv_pages, dtype=np.float64)
    n_tok, hq, lkv = qn.shape
    rope = qp.shape[2]
    assert lkv == kv_lora_rank and rope == qk_rope_head_dim
    off = -(-lkv // 128) * 128
    pg = pages.shape[1]
    scale = float(lkv + rope) ** -0.5 if softmax_scale is None else float(softmax_scale)
    bt = np.asarray(block_tables).reshape(len(context_lens), -1)
    out = np.zeros((n_tok, hq, lkv), dtype=np.float64)
    sinks = None if softmax_aux is None else np.asarray(softmax_aux, dtype=np.float64).reshape(-1)
    for i in range(int(np.asarray(num_seqs).reshape(-1)[0])):
        q0, q1 = int(query_start_loc[i]), int(query_start_loc[i + 1])
        ctx, q_len = int(context_lens[i]), q1 - q0
        if q_len <= 0 or ctx <= 0:
            continue
        n_pages = -(-ctx // pg)
        seq = pages[bt[i, :n_pages]].reshape(n_pages * pg, -1)[:ctx]
        latent, k_pe = seq[:, :lkv], seq[:, off:off + rope]
        pos = ctx - q_len + np.arange(q_len)
        j = np.arange(ctx)
        visible = j[None, :] <= pos[:, None]
        if sliding_window is not None and int(sliding_window) > 0:
            visible &= j[None, :] > (pos[:, None] - int(sliding_window))
        for h in range(hq):
            s = (qn[q0:q1, h, :] @ latent.T + qp[q0:q1, h, :] @ k_pe.T) * scale
            if logits_soft_cap is not None and float(logits_soft_cap) > 0:
                s = float(logits_soft_cap) * np.tanh(s / float(logits_soft_cap))
            s = np.where(visible, s, -np.inf)
            m = s.max(axis=1, keepdims=True)
            if sinks is not None:
                m = np.maximum(m, sinks[h])
            m = np.where(np.isfinite(m), m, 0.0)
            p = np.exp(s - m)
            denom = p.sum(axis=1, keepdims=True)
            if sinks is not None:
                denom = denom + np.exp(sinks[h] - m)
            out[q0:q1, h, :] = (p @ latent) / np.where(denom > 0, denom, 1.0)
    return out
