"""Pins the oracle's integer / scatter functions on the reference's own test vectors."""

import numpy as np
import pytest

from rpa_testlib import orc


def test_reference_vector_slice_mapping():
    # /root/reference/tests/layers/caching/test_kv_cache_update_jax.py:84-119
    rng = np.random.default_rng(0)
    new_tokens = rng.standard_normal((16, 4, 8), dtype=np.float32)
    cache = np.zeros((64, 4, 8), dtype=np.float32)
    lens = np.array([3, 2, 2, 0, 0], dtype=np.int32)
    src = np.concatenate(([0], np.cumsum(lens[:-1], dtype=np.int32))).astype(np.int32)
    dst = np.array([10, 20, 30, 0, 0], dtype=np.int32)
    updated = orc.kv_cache_update_ref(new_tokens, np.stack([dst, src, lens]), cache, [3], page_size=4)
    expected = np.zeros_like(cache)
    for i in range(3):
        expected[dst[i]:dst[i] + lens[i]] = new_tokens[src[i]:src[i] + lens[i]]
    np.testing.assert_allclose(updated, expected, atol=0.0, rtol=0.0)


def test_reference_vector_localize_zeroes_non_local():
    # test_kv_cache_update_jax.py:122-146
    si = np.array([[0, 5, 8, 13], [0, 1, 2, 4], [1, 1, 2, 1]], dtype=np.int32)
    got = orc.localize_slice_indices_ref(si, [4], page_size=4, local_flat_cache_positions=8, page_shard_index=1)
    np.testing.assert_array_equal(got, np.array([[0, 0, 0, 5], [0, 0, 2, 4], [0, 0, 2, 1]], dtype=np.int32))


def test_reference_vector_page_shard_local_offsets():
    # test_kv_cache_update_jax.py:149-180
    cache = np.zeros((8, 2, 4), dtype=np.float32)
    new_tokens = np.arange(6 * 2 * 4, dtype=np.float32).reshape(6, 2, 4)
    si = np.array([[0, 8, 12, 0], [0, 2, 4, 0], [2, 2, 2, 0]], dtype=np.int32)
    updated = orc.kv_cache_update_ref(new_tokens, si, cache, [3], page_size=4, page_shard_index=1)
    expected = np.zeros_like(cache)
    expected[0:2] = new_tokens[2:4]
    expected[4:6] = new_tokens[4:6]
    np.testing.assert_allclose(updated, expected, atol=0.0, rtol=0.0)


@pytest.mark.parametrize("scheduled,context_lens,expected", [([4], [4], [0, 1, 1]), ([4, 1, 0], [4, 9, 0], [1, 2, 2])])
def test_reference_vector_request_distribution(scheduled, context_lens, expected):
    # /root/reference/tests/inference/test_request_distribution_bounds.py:31-44
    np.testing.assert_array_equal(orc.request_distribution_ref(scheduled, context_lens), np.array(expected, dtype=np.int32))


def test_reference_vector_host_builder_distribution():
    # test_request_distribution_bounds.py:47-58: scheduled [4,1,0,0], computed [0,8,0,0] -> seq_lens [4,9,0,0] -> [1,2,2]
    scheduled = np.array([4, 1, 0, 0]); computed = np.array([0, 8, 0, 0])
    np.testing.assert_array_equal(orc.request_distribution_ref(scheduled, computed + scheduled), [1, 2, 2])


def test_reference_vector_storage_layout():
    # /root/reference/tests/layers/caching/test_ragged_page_dtype_compat.py:34-60 and cache.py:143-158, 616-647
    assert orc.storage_layout_ref(8, 128, 16) == {"packing": 2, "combined": 16, "groups": 8, "head_dim": 128}
    lay = orc.storage_layout_ref(4, 128, 8)
    assert (lay["packing"], lay["combined"], lay["groups"]) == (4, 8, 2)
    assert orc.storage_layout_ref(2, 64, 32) == {"packing": 1, "combined": 2, "groups": 2, "head_dim": 128}
    assert orc.storage_layout_ref(8, 256, 16)["head_dim"] == 256
    assert orc.storage_layout_ref(8, 96, 16)["head_dim"] == 128


def test_slot_mapping_closed_form_and_round_trip():
    rng = np.random.default_rng(1)
    pg, n_req, max_pages = 16, 9, 12
    scheduled = np.array([1, 1, 37, 0, 80, 1, 16, 50, 3], dtype=np.int32)
    computed = np.array([5, 15, 0, 9, 3, 31, 16, 100, 29], dtype=np.int32)
    table = rng.permutation(np.arange(1, n_req * max_pages + 1)).reshape(n_req, max_pages).astype(np.int32)
    si, total = orc.slot_mapping_v2_ref(scheduled, computed, table, pg, slices_per_page=8)
    assert si.shape[1] % 8 == 0 and si[2, total:].sum() == 0
    # closed form: scheduled token k of request r (absolute position t) lands at table[r, t // pg] * pg + t % pg
    want_dst, want_src, src = [], [], 0
    for r in range(n_req):
        for t in range(computed[r], computed[r] + scheduled[r]):
            want_dst.append(table[r, t // pg] * pg + t % pg)
            want_src.append(src)
            src += 1
    got_dst = np.concatenate([np.arange(si[0, c], si[0, c] + si[2, c]) for c in range(total)])
    got_src = np.concatenate([np.arange(si[1, c], si[1, c] + si[2, c]) for c in range(total)])
    np.testing.assert_array_equal(got_dst, want_dst)
    np.testing.assert_array_equal(got_src, want_src)
    assert len(set(got_dst.tolist())) == len(got_dst) == scheduled.sum()
    # slices never straddle a page
    assert np.all(si[0, :total] // pg == (si[0, :total] + si[2, :total] - 1) // pg)
    # round trip through the scatter: every scheduled token readable at its closed-form slot
    T = int(scheduled.sum()) + 5
    new_kv = rng.standard_normal((T, 2, 4), dtype=np.float32)
    pages = np.zeros(((n_req * max_pages + 1) * pg, 2, 4), dtype=np.float32)
    out = orc.kv_cache_update_ref(new_kv, si, pages, [total], page_size=pg)
    np.testing.assert_array_equal(out[want_dst], new_kv[want_src])
    assert np.count_nonzero(out.reshape(len(out), -1).any(axis=1)) == scheduled.sum()


def test_ragged_scatter_equals_slice_scatter():
    # the fused v3 write must place tokens exactly where the v2 slot mapping does
    rng = np.random.default_rng(2)
    pg, hkv, d = 16, 3, 8
    scheduled = np.array([1, 8, 33, 0, 1], dtype=np.int32)
    computed = np.array([16, 122, 222, 7, 0], dtype=np.int32)
    ctx = computed + scheduled
    ctx[3] = 0
    table = rng.permutation(np.arange(1, 5 * 20 + 1)).reshape(5, 20).astype(np.int32)
    qsl = np.concatenate([[0], np.cumsum(scheduled)]).astype(np.int32)
    T = int(qsl[-1])
    key = rng.standard_normal((T, hkv, d), dtype=np.float32)
    val = rng.standard_normal((T, hkv, d), dtype=np.float32)
    pages = rng.standard_normal((101, pg, 2 * hkv, d), dtype=np.float32)
    got = orc.page_scatter_ragged_ref(key, val, pages, ctx, table, qsl, [5])
    si, total = orc.slot_mapping_v2_ref(scheduled, computed, table, pg)
    new_kv = np.stack([key, val], axis=2).reshape(T, 2 * hkv, d)  # cache.py:928
    want = orc.kv_cache_update_ref(new_kv, si, pages.reshape(-1, 2 * hkv, d), [total], page_size=pg).reshape(pages.shape)
    np.testing.assert_array_equal(got, want)


def test_scatter_drop_rules():
    new_kv = np.arange(6 * 2, dtype=np.float32).reshape(6, 2, 1) + 1
    pages = np.zeros((16, 2, 1), dtype=np.float32)
    # column 2 points past the cache (dropped), column 3 runs its source off the end (tail dropped)
    si = np.array([[2, 14, 100, 6], [0, 2, 0, 5], [2, 4, 1, 3]], dtype=np.int32)
    out = orc.kv_cache_update_ref(new_kv, si, pages, [4], page_size=4)
    np.testing.assert_array_equal(out[2:4], new_kv[0:2])
    np.testing.assert_array_equal(out[14:16], new_kv[2:4])  # positions 16, 17 fall off the cache
    assert out[6, 0, 0] == 0  # packed tokens 6.. are beyond the 6 source rows the scatter can address
    assert orc.kv_cache_update_ref(new_kv, si, pages, [0], page_size=4).sum() == 0
    empty = orc.kv_cache_update_ref(new_kv, si, np.zeros((0, 2, 1), np.float32), [4], page_size=4)
    assert empty.shape == (0, 2, 1)
