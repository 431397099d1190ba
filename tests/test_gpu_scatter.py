"""GPU parity: page scatter kernels (through the C ABI) are bit-exact against the oracle and the
reference's own test vectors (tests/layers/caching/test_kv_cache_update_jax.py)."""

import numpy as np
import pytest

import rpa_testlib as tl
from rpa_testlib import BF16, F32, FP8, orc

pytestmark = pytest.mark.gpu


def _scatter_slices(gpu, new_kv, si, pages, n_valid, page_size, shard=0):
    import torch
    from easydel_amd import kernels

    d_new = torch.from_numpy(new_kv).to(gpu)
    d_pages = torch.from_numpy(pages.copy()).to(gpu)
    d_si = torch.from_numpy(np.ascontiguousarray(si, dtype=np.int32)).to(gpu)
    d_n = torch.tensor([n_valid], dtype=torch.int32, device=gpu)
    kernels.page_scatter_slices(d_new, d_si, d_n, d_pages, page_size=page_size, page_shard_index=shard)
    torch.cuda.synchronize()
    return d_pages.cpu().numpy()


def test_reference_vector_slice_mapping(gpu):
    # test_kv_cache_update_jax.py:84-119
    rng = np.random.default_rng(0)
    new_tokens = rng.standard_normal((16, 4, 8), dtype=np.float32)
    cache = np.zeros((64, 4, 8), dtype=np.float32)
    lens = np.array([3, 2, 2, 0, 0], dtype=np.int32)
    src = np.concatenate(([0], np.cumsum(lens[:-1], dtype=np.int32))).astype(np.int32)
    dst = np.array([10, 20, 30, 0, 0], dtype=np.int32)
    got = _scatter_slices(gpu, new_tokens, np.stack([dst, src, lens]), cache, 3, page_size=4)
    expected = np.zeros_like(cache)
    for i in range(3):
        expected[dst[i]:dst[i] + lens[i]] = new_tokens[src[i]:src[i] + lens[i]]
    assert np.array_equal(got, expected)


def test_reference_vector_page_shard_local_offsets(gpu):
    # test_kv_cache_update_jax.py:149-180
    cache = np.zeros((8, 2, 4), dtype=np.float32)
    new_tokens = np.arange(6 * 2 * 4, dtype=np.float32).reshape(6, 2, 4)
    si = np.array([[0, 8, 12, 0], [0, 2, 4, 0], [2, 2, 2, 0]], dtype=np.int32)
    got = _scatter_slices(gpu, new_tokens, si, cache, 3, page_size=4, shard=1)
    expected = np.zeros_like(cache)
    expected[0:2] = new_tokens[2:4]
    expected[4:6] = new_tokens[4:6]
    assert np.array_equal(got, expected)


@pytest.mark.parametrize("dtype,C,D", [(np.float32, 4, 8), (np.uint16, 16, 128), (np.uint8, 16, 128), (np.uint16, 3, 5)])
def test_slices_random_against_oracle(gpu, dtype, C, D):
    rng = np.random.default_rng(3)
    T, page_size, n_pages = 300, 16, 40
    scheduled = np.array([1, 1, 37, 0, 80, 1, 16, 50], dtype=np.int32)
    computed = np.array([5, 15, 0, 9, 3, 31, 16, 100], dtype=np.int32)
    table = rng.permutation(np.arange(1, n_pages))[: 8 * 4].reshape(8, 4)[:, :].astype(np.int32)
    table = np.concatenate([table, rng.permutation(np.arange(1, n_pages))[:32].reshape(8, 4).astype(np.int32)], axis=1)
    # make the tables collision free across requests
    table = rng.permutation(np.arange(1, 8 * 10 + 1)).reshape(8, 10).astype(np.int32)
    si, total = orc.slot_mapping_v2_ref(scheduled, computed, table, page_size, slices_per_page=8)
    n_pages = 8 * 10 + 1
    if dtype == np.float32:
        new_kv = rng.standard_normal((T, C, D), dtype=np.float32)
        pages = rng.standard_normal((n_pages * page_size, C, D), dtype=np.float32)
    else:
        info = np.iinfo(dtype)
        new_kv = rng.integers(0, info.max, size=(T, C, D), dtype=dtype)
        pages = rng.integers(0, info.max, size=(n_pages * page_size, C, D), dtype=dtype)
    want = orc.kv_cache_update_ref(new_kv, si, pages, [total], page_size=page_size)
    got = _scatter_slices(gpu, new_kv, si, pages, total, page_size=page_size)
    assert np.array_equal(got, want)
    assert not np.array_equal(got, pages)
    # each shard of a 3-way page split applies exactly its local slices
    local = (n_pages // 3) * page_size
    for shard in range(3):
        part = pages[shard * local:(shard + 1) * local]
        want_s = orc.kv_cache_update_ref(new_kv, si, part, [total], page_size=page_size, page_shard_index=shard)
        got_s = _scatter_slices(gpu, new_kv, si, part, total, page_size=page_size, shard=shard)
        assert np.array_equal(got_s, want_s)


def test_slices_drop_rules(gpu):
    # inactive columns, out-of-range destinations and sources, packed tokens beyond T
    new_kv = np.arange(6 * 2 * 4, dtype=np.float32).reshape(6, 2, 4) + 1
    pages = np.zeros((16, 2, 4), dtype=np.float32)
    si = np.array([[2, 14, 100, 6, 9], [0, 2, 0, 5, 1], [2, 4, 1, 3, 1]], dtype=np.int32)
    for n_valid in (0, 1, 3, 4, 5):
        want = orc.kv_cache_update_ref(new_kv, si, pages, [n_valid], page_size=4)
        got = _scatter_slices(gpu, new_kv, si, pages, n_valid, page_size=4)
        assert np.array_equal(got, want), n_valid


def test_empty_inputs_are_noops(gpu):
    import torch
    from easydel_amd import kernels

    pages = torch.zeros((8, 2, 4), device=gpu)
    out = kernels.page_scatter_slices(torch.zeros((0, 2, 4), device=gpu), torch.zeros((3, 4), dtype=torch.int32, device=gpu),
                                      torch.zeros(1, dtype=torch.int32, device=gpu), pages, page_size=4)
    assert out is pages and float(pages.abs().sum()) == 0.0


@pytest.mark.parametrize("kv_dtype,Hkv,D,page_size", [(BF16, 8, 128, 64), (F32, 2, 64, 16), (FP8, 8, 128, 64), (BF16, 3, 80, 16)])
def test_ragged_scatter_against_oracle(gpu, kv_dtype, Hkv, D, page_size):
    import torch
    from easydel_amd import kernels

    ctx = [17, 64, 130, 255, 1, 90]
    q_lens = [1, 1, 8, 33, 1, 90]
    b = tl.make_batch(21, ctx, q_lens, Hq=Hkv, Hkv=Hkv, D=D, page_size=page_size, kv_dtype=kv_dtype, pad_rows=2, pad_tokens=3)
    rng = np.random.default_rng(5)
    dt = b.kv_raw.dtype
    if dt == np.float32:
        key = rng.standard_normal((b.T, Hkv, D), dtype=np.float32)
        val = rng.standard_normal((b.T, Hkv, D), dtype=np.float32)
    else:
        key = rng.integers(0, np.iinfo(dt).max, size=(b.T, Hkv, D), dtype=dt)
        val = rng.integers(0, np.iinfo(dt).max, size=(b.T, Hkv, D), dtype=dt)
    want = orc.page_scatter_ragged_ref(key, val, b.kv_raw, b.context_lens, b.block_tables, b.query_start_loc, b.num_seqs)
    d = tl.device_batch(b, gpu)
    kernels.page_scatter_ragged(tl.to_torch(key, kv_dtype, gpu), tl.to_torch(val, kv_dtype, gpu), d["kv_pages"],
                                d["context_lens"], d["block_tables"], d["query_start_loc"], d["num_seqs"])
    torch.cuda.synchronize()
    got = d["kv_pages"].view(torch.uint8).cpu().numpy()
    assert np.array_equal(got, want.view(np.uint8).reshape(got.shape))
    assert not np.array_equal(got, b.kv_raw.view(np.uint8).reshape(got.shape))


def test_fused_v3_equals_scatter_then_attend(gpu):
    import torch
    from easydel_amd import kernels

    ctx = [17, 64, 130, 255, 700]
    q_lens = [1, 1, 8, 33, 1]
    b = tl.make_batch(22, ctx, q_lens, Hq=32, Hkv=8, D=128, page_size=64, pad_rows=1)
    rng = np.random.default_rng(6)
    key = orc.f32_to_bf16_bits(rng.standard_normal((b.T, 8, 128), dtype=np.float32))
    val = orc.f32_to_bf16_bits(rng.standard_normal((b.T, 8, 128), dtype=np.float32))
    pages_after = orc.page_scatter_ragged_ref(key, val, b.kv_raw, b.context_lens, b.block_tables, b.query_start_loc, b.num_seqs)
    want = tl.oracle_out(b, kv_val=orc.bf16_bits_to_f32(pages_after).astype(np.float64))
    d = tl.device_batch(b, gpu)
    dist = torch.tensor(orc.request_distribution_ref(q_lens + [0], b.context_lens), dtype=torch.int32, device=gpu)
    # the v3 page buffer shape [P, pg, groups, packing, D] is the same bytes as [P, pg, 2*Hkv, D]
    pages5 = d["kv_pages"].view(b.P, 64, 8, 2, 128)
    out, pages_out = kernels.ragged_paged_attention_v3(
        d["query"], tl.to_torch(key, BF16, gpu), tl.to_torch(val, BF16, gpu), pages5, d["context_lens"],
        d["block_tables"].reshape(-1), d["query_start_loc"], dist)
    torch.cuda.synchronize()
    assert pages_out is pages5
    assert np.array_equal(pages5.view(torch.int16).cpu().numpy().view(np.uint16).reshape(pages_after.shape), pages_after)
    tl.assert_close(tl.from_torch(out, BF16), want, b, "fused v3")
