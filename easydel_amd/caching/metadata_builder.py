"""Host-side (numpy) builders of the per-step integer metadata.

Restates, as plain loops, what the reference computes in ``easydel/caching/_metadatabuilder.py:783-1020`` and
``easydel/inference/esurge/runners/executors/batch_preparer.py:612-709``: which slices of the new K/V go to
which cache positions (v2), the decode / prefill / total request counts (v3), and the padded ragged arrays.
These run on the host once per step; they feed the kernels and are not kernels themselves.
"""

from __future__ import annotations

import numpy as np


def request_distribution(scheduled, context_lens) -> np.ndarray:
    """``[decode_end, prefill_end, total]``: a row is a decode row when it schedules one token onto a
    context longer than one (reference ``ragged_page_attention.py:177-187``)."""
    scheduled = np.asarray(scheduled, dtype=np.int32)
    context_lens = np.asarray(context_lens, dtype=np.int32)
    has_tokens = scheduled > 0
    is_decode = (scheduled == 1) & (context_lens > 1) & has_tokens
    decode = int(is_decode.sum())
    return np.array([decode, decode + int((has_tokens & ~is_decode).sum()), int(has_tokens.sum())], dtype=np.int32)


def compute_slot_mapping_v2(*, num_requests: int, scheduled, num_computed_tokens, page_table, page_size: int,
                            max_pages_per_req: int | None = None, slices_per_page: int = 1,
                            max_padded_slices: int | None = None):
    """One ``(cache_start, new_kv_start, length)`` slice per (request, page touched), padded to a multiple of
    ``slices_per_page`` (reference ``_metadatabuilder.py:783-882``).  Returns ``(slot_mapping[3, n], total)``."""
    if num_requests <= 0:
        return np.zeros((3, 1), dtype=np.int32), 0
    scheduled = np.asarray(scheduled)[:num_requests].astype(np.int64)
    computed = np.asarray(num_computed_tokens)[:num_requests].astype(np.int64)
    page_table = np.asarray(page_table)
    cols, src = [], 0
    for r in range(num_requests):
        n = int(scheduled[r])
        if n <= 0:
            continue
        start, end = int(computed[r]), int(computed[r]) + n
        for page_idx in range(start // page_size, (end - 1) // page_size + 1):
            lo, hi = max(start, page_idx * page_size), min(end, (page_idx + 1) * page_size)
            col = min(page_idx, (max_pages_per_req or page_table.shape[1]) - 1)
            cols.append((int(page_table[r, col]) * page_size + lo % page_size, src, hi - lo))
            src += hi - lo
    total = len(cols)
    if total == 0:
        return np.zeros((3, 1), dtype=np.int32), 0
    padded = cdiv(total, slices_per_page) * slices_per_page
    if max_padded_slices is not None:
        padded = min(int(max_padded_slices), padded)
    padded = max(padded, 1)
    out = np.zeros((3, padded), dtype=np.int32)
    keep = min(total, padded)
    out[:, :keep] = np.asarray(cols[:keep], dtype=np.int32).T
    return out, total


def cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


def compute_ragged_batch_fields(*, scheduled_full, active_mask_full, num_computed_tokens, page_table, version: str,
                                max_num_reqs: int, page_size: int = 128, slices_per_page: int = 1) -> dict:
    """The arrays of ``RaggedPagesMetadata`` for one step, with the reference's padding conventions: rows past
    the live requests are zero, ``query_start_loc`` is extended flat, ``context_lens`` is zero where nothing is
    scheduled (``batch_preparer.py:612-709``), the page-table pad value is the null page 0."""
    scheduled = np.asarray(scheduled_full, dtype=np.int32)[:max_num_reqs].copy()
    active = np.asarray(active_mask_full, dtype=bool)[:max_num_reqs]
    computed = np.asarray(num_computed_tokens, dtype=np.int32)[:max_num_reqs]
    scheduled[~active] = 0
    live = np.nonzero(scheduled > 0)[0]
    num_requests = int(live.max()) + 1 if live.size else 0
    qsl = np.zeros(max_num_reqs + 1, dtype=np.int32)
    qsl[1:] = np.cumsum(scheduled)
    context_lens = np.where(scheduled > 0, computed + scheduled, 0).astype(np.int32)
    fields = {
        "pages_tables": np.asarray(page_table, dtype=np.int32)[:max_num_reqs],
        "context_lens": context_lens,
        "query_start_loc": qsl,
        "num_seqs": np.array([num_requests], dtype=np.int32),
        "position_ids": np.concatenate([computed[r] + np.arange(scheduled[r]) for r in range(max_num_reqs)] or [[]]).astype(np.int32),
    }
    if version == "v3":
        dist = request_distribution(scheduled, context_lens)
        dist[2] = num_requests  # the host builders put the live row count in slot 2 (_metadatabuilder.py:983-991)
        fields["request_distribution"] = dist
    else:
        slot_mapping, total = compute_slot_mapping_v2(num_requests=num_requests, scheduled=scheduled,
                                                      num_computed_tokens=computed, page_table=page_table,
                                                      page_size=page_size, slices_per_page=slices_per_page)
        fields["slot_mapping"] = slot_mapping
        fields["num_kv_update_slices"] = np.array([total], dtype=np.int32)
    return fields
