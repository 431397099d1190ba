"""The oracle's statement of one data-parallel rank's share of the page-sharded attention (reference
easydel/operations/kernels/ragged_page_attention.py:645-717), pinned by what the scheme has to guarantee."""

import numpy as np
import pytest

from oracle import rpa_oracle as orc


def _sharded_batch(seed, n_shards, rows_per_shard, local_pages, page_size=16, Hq=4, Hkv=2, D=16):
    """Sequences whose pages live on the shard of their metadata row; every shard's rows are live first, then padding."""
    rng = np.random.default_rng(seed)
    S = n_shards * rows_per_shard
    M = 6
    ctx = np.zeros(S, np.int32)
    q_lens = np.zeros(S, np.int32)
    tables = np.zeros((S, M), np.int32)
    for sh in range(n_shards):
        live = int(rng.integers(1, rows_per_shard + 1))
        free = list(rng.permutation(np.arange(1 if sh == 0 else 0, local_pages)) + sh * local_pages)
        for r in range(live):
            i = sh * rows_per_shard + r
            ctx[i] = int(rng.integers(1, M * page_size + 1))
            q_lens[i] = int(rng.integers(1, min(int(ctx[i]), 9) + 1))
            need = -(-int(ctx[i]) // page_size)
            tables[i, :need] = [free.pop() for _ in range(need)]
    # query_start_loc over all rows in order (rows without tokens have empty spans)
    qsl = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    T = int(qsl[-1])
    P = n_shards * local_pages
    kv = rng.standard_normal((P, page_size, 2 * Hkv, D))
    q = rng.standard_normal((T, Hq, D))
    return dict(S=S, T=T, P=P, ctx=ctx, q_lens=q_lens, tables=tables, qsl=qsl, kv=kv, q=q, page_size=page_size, Hkv=Hkv)


@pytest.mark.parametrize("seed,n_shards", [(0, 2), (1, 4), (2, 3)])
def test_sum_over_ranks_equals_the_global_attention(seed, n_shards):
    b = _sharded_batch(seed, n_shards, rows_per_shard=3, local_pages=24)
    # rows are live in the order the reference needs (live rows first) only per shard, not globally: the global call
    # therefore counts every row, live or not, and empty rows contribute nothing
    want = orc.ragged_paged_attention_ref(b["q"], b["kv"], b["ctx"], b["tables"], b["qsl"], np.array([b["S"]], np.int32))
    total = np.zeros_like(want)
    owned = np.zeros(b["T"], dtype=int)
    for sh in range(n_shards):
        m = orc.dp_local_shard_ref(sh, n_shards, b["ctx"], b["tables"], b["qsl"], 24, b["T"])
        local_kv = b["kv"][sh * 24:(sh + 1) * 24]
        rows = b["S"] // n_shards
        out = orc.ragged_paged_attention_ref(b["q"], local_kv, m["context_lens"], m["block_tables"].reshape(rows, -1),
                                             m["query_start_loc"], m["distribution"][2:3])
        out = np.where(m["token_mask"][:, None, None], out, 0.0)
        total += out.astype(np.float32)
        owned += m["token_mask"]
    assert np.array_equal(owned, np.ones(b["T"], dtype=int)), "every scheduled token belongs to exactly one rank"
    assert np.abs(total - want).max() < 1e-5


def test_rebasing_and_clipping_of_page_ids():
    tables = np.array([[0, 5, 9], [10, 19, 0], [20, 25, 29], [3, 0, 0]], np.int32)
    ctx = np.array([40, 30, 45, 7], np.int32)
    qsl = np.array([0, 1, 2, 10, 11], np.int32)
    m0 = orc.dp_local_shard_ref(0, 2, ctx, tables, qsl, 10, 11)
    m1 = orc.dp_local_shard_ref(1, 2, ctx, tables, qsl, 10, 11)
    # shard 0 owns pages 0..9: its own ids stay, foreign ones clip to the pool's ends
    assert m0["block_tables"].tolist() == [0, 5, 9, 9, 9, 0]
    # shard 1 owns pages 10..19: 20.. clip to 9, ids below 10 clip to 0
    assert m1["block_tables"].tolist() == [9, 9, 9, 0, 0, 0]
    assert m0["query_start_loc"].tolist() == [0, 1, 2] and m1["query_start_loc"].tolist() == [2, 10, 11]
    assert m0["distribution"].tolist() == [2, 2, 2] and m1["distribution"].tolist() == [1, 2, 2]
    assert m0["token_mask"].tolist() == [True, True] + [False] * 9
    assert m1["token_mask"].tolist() == [False, False] + [True] * 9
    with pytest.raises(ValueError):
        orc.dp_local_shard_ref(0, 3, ctx, tables, qsl, 10, 11)
