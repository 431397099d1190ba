"""One data-parallel rank's share of the page-sharded attention (reference
easydel/operations/kernels/ragged_page_attention.py:645-717) on one GPU: the ranks' calls run one after the other on
their slices of the pool, their outputs are summed as the reference's psum does, and the result is compared with the
oracle's statement of the same scheme and with one call over the whole pool."""

import numpy as np
import pytest
import torch

import rpa_testlib as tl
from easydel_amd import kernels
from easydel_amd.caching import RaggedPagesMetadata
from easydel_amd.operations import OperationMetadata, OperationRegistry
from easydel_amd.operations.ragged_page_attention import dp_local_reduce
from rpa_testlib import BF16, FP8, INT8, orc

pytestmark = pytest.mark.gpu


def _sharded_batch(seed, n_shards, rows_per_shard, local_pages, page_size, Hq, Hkv, D):
    rng = np.random.default_rng(seed)
    S, M = n_shards * rows_per_shard, 40
    ctx, q_lens, tables = np.zeros(S, np.int32), np.zeros(S, np.int32), np.zeros((S, M), np.int32)
    kinds = [(1, 1), (1, 1), (3, 3), (40, 200), (1, 1), (130, 700)]  # (q_len, least context)
    for sh in range(n_shards):
        live = int(rng.integers(2, rows_per_shard + 1))
        free = list(rng.permutation(np.arange(1 if sh == 0 else 0, local_pages)) + sh * local_pages)
        for r in range(live):
            i = sh * rows_per_shard + r
            ql, lo = kinds[int(rng.integers(0, len(kinds)))]
            ctx[i] = int(rng.integers(max(lo, ql), M * page_size + 1))
            q_lens[i] = ql
            need = -(-int(ctx[i]) // page_size)
            tables[i, :need] = [free.pop() for _ in range(need)]
    qsl = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    T, P = int(qsl[-1]), n_shards * local_pages
    raw = lambda *shape: orc.f32_to_bf16_bits(rng.standard_normal(shape, dtype=np.float32))  # noqa: E731
    return dict(S=S, T=T, P=P, M=M, ctx=ctx, q_lens=q_lens, tables=tables, qsl=qsl, pages=raw(P, page_size, 2 * Hkv, D),
                q=raw(T, Hq, D), k=raw(T, Hkv, D), v=raw(T, Hkv, D))


@pytest.mark.parametrize("n_shards,page_size,Hq,Hkv,D", [(2, 64, 32, 8, 128), (4, 32, 8, 2, 64)])
def test_dp_local_shards_sum_to_the_global_result(gpu, n_shards, page_size, Hq, Hkv, D):
    local_pages = 400
    b = _sharded_batch(70 + n_shards, n_shards, 5, local_pages, page_size, Hq, Hkv, D)
    up = lambda a: torch.from_numpy(a).to(gpu)  # noqa: E731
    meta = RaggedPagesMetadata(pages_tables=up(b["tables"]), context_lens=up(b["ctx"]), query_start_loc=up(b["qsl"]),
                               num_seqs=torch.tensor([b["S"]], dtype=torch.int32, device=gpu),
                               request_distribution=up(orc.request_distribution_ref(b["q_lens"], b["ctx"])), page_size=page_size)
    q, k, v = (tl.to_torch(b[x], BF16, gpu) for x in ("q", "k", "v"))
    pool = tl.to_torch(b["pages"], BF16, gpu)
    op = OperationRegistry.create("ragged_page_attention_v3", OperationMetadata())
    outs, new_pages = [], []
    for sh in range(n_shards):
        out, pages = op.forward_v3_dp_local_shard(q, k, v, pool[sh * local_pages:(sh + 1) * local_pages].clone(), meta, sh, n_shards)
        torch.cuda.synchronize()
        m = orc.dp_local_shard_ref(sh, n_shards, b["ctx"], b["tables"], b["qsl"], local_pages, b["T"])
        got = tl.from_torch(out, BF16)
        assert not np.abs(got[~m["token_mask"]]).any(), f"shard {sh}: rows of other ranks' tokens must be zero"
        outs.append(out)
        new_pages.append(pages)
    total = tl.from_torch(dp_local_reduce(outs), BF16)
    # the page write: every rank wrote its own sequences' tokens; together they are the global write
    want_pages = orc.page_scatter_ragged_ref(b["k"], b["v"], b["pages"], b["ctx"], b["tables"], b["qsl"], [b["S"]])
    got_pages = torch.cat(new_pages).view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(got_pages, want_pages)
    want = orc.ragged_paged_attention_ref(orc.bf16_bits_to_f32(b["q"]).astype(np.float64), orc.bf16_bits_to_f32(want_pages).astype(np.float64),
                                          b["ctx"], b["tables"], b["qsl"], [b["S"]])
    err = np.abs(total - want)
    assert err.max() <= tl.TOL_BF16_MAX and err.mean() <= tl.TOL_BF16_MEAN, (err.max(), err.mean())
    # and one call over the whole pool gives the same rows within the same bound (every row counted: the live rows
    # of the ranks are not contiguous in the global arrays, rows without tokens are skipped by their empty spans)
    every_row = torch.tensor([0, 0, b["S"]], dtype=torch.int32, device=gpu)
    out_global, _ = kernels.ragged_paged_attention_v3(q, k, v, pool.clone(), meta.context_lens, meta.pages_tables.reshape(-1),
                                                      meta.query_start_loc, every_row)
    torch.cuda.synchronize()
    assert np.abs(tl.from_torch(out_global, BF16) - want).max() <= tl.TOL_BF16_MAX
    with pytest.raises(ValueError):
        op.forward_v3_dp_local_shard(q, k, v, pool[:local_pages], meta, 0, 3 if b["S"] % 3 else 7)


@pytest.mark.parametrize("kv_dtype", [INT8, FP8])
def test_dp_local_shards_of_a_scaled_8bit_pool(gpu, kv_dtype):
    """A rank's share of a scaled 8-bit pool travels with its rows of the scales: the rank's write quantises into its
    pages and scales, the ranks' outputs sum to the attention over the dequantised global pool, and int8 pages
    without scales are refused."""
    n_shards, local_pages, page_size, Hq, Hkv, D = 2, 400, 64, 32, 8, 128
    b = _sharded_batch(75, n_shards, 5, local_pages, page_size, Hq, Hkv, D)
    rng = np.random.default_rng(76)
    P = b["P"]
    # pages that already hold context: codes and per-(page, combined head) scales
    codes = rng.integers(0, 255, size=(P, page_size, 2 * Hkv, D), dtype=np.uint8)
    if kv_dtype == FP8:
        codes[(codes & 0x7f) == 0x7f] = 0x3c  # no NaN codes in the stale contents
    hi = 0.03 if kv_dtype == INT8 else 0.008  # the largest code is 127 / 448: stored values stay within a few units
    scales = rng.uniform(hi / 3, hi, size=(P, 2 * Hkv)).astype(np.float32)
    up = lambda a: torch.from_numpy(a).to(gpu)  # noqa: E731
    meta = RaggedPagesMetadata(pages_tables=up(b["tables"]), context_lens=up(b["ctx"]), query_start_loc=up(b["qsl"]),
                               num_seqs=torch.tensor([b["S"]], dtype=torch.int32, device=gpu),
                               request_distribution=up(orc.request_distribution_ref(b["q_lens"], b["ctx"])), page_size=page_size)
    q, k, v = (tl.to_torch(b[x], BF16, gpu) for x in ("q", "k", "v"))
    torch_kv = {FP8: torch.float8_e4m3fn, INT8: torch.int8}[kv_dtype]
    pool = up(codes).view(torch_kv)
    pool_scales = up(scales)
    op = OperationRegistry.create("ragged_page_attention_v3", OperationMetadata())
    outs, new_codes, new_scales = [], [], []
    for sh in range(n_shards):
        rows = slice(sh * local_pages, (sh + 1) * local_pages)
        out, pages, sc = op.forward_v3_dp_local_shard(q, k, v, pool[rows].clone(), meta, sh, n_shards,
                                                      local_kv_scales=pool_scales[rows].clone(), num_kv_heads=Hkv)
        torch.cuda.synchronize()
        m = orc.dp_local_shard_ref(sh, n_shards, b["ctx"], b["tables"], b["qsl"], local_pages, b["T"])
        assert not np.abs(tl.from_torch(out, BF16)[~m["token_mask"]]).any(), f"shard {sh}: rows of other ranks' tokens must be zero"
        outs.append(out)
        new_codes.append(pages.view(torch.uint8).cpu().numpy())
        new_scales.append(sc.cpu().numpy())
    # the ranks' writes together are the global quantising write, bit for bit
    want_codes, want_scales = orc.page_scatter_ragged_quantised_ref(orc.bf16_bits_to_f32(b["k"]), orc.bf16_bits_to_f32(b["v"]), codes, scales,
                                                                    b["ctx"], b["tables"], b["qsl"], [b["S"]], kv_dtype=kv_dtype)
    assert np.array_equal(np.concatenate(new_scales), want_scales)
    assert np.array_equal(np.concatenate(new_codes).reshape(want_codes.shape), want_codes)
    kv_val = orc.decode_codes(want_codes, kv_dtype).astype(np.float64) * want_scales[:, None, :, None]
    want = orc.ragged_paged_attention_ref(orc.bf16_bits_to_f32(b["q"]).astype(np.float64), kv_val, b["ctx"], b["tables"], b["qsl"], [b["S"]])
    err = np.abs(tl.from_torch(dp_local_reduce(outs), BF16) - want)
    assert err.max() <= tl.TOL_BF16_MAX and err.mean() <= tl.TOL_BF16_MEAN, (err.max(), err.mean())
    if kv_dtype == INT8:
        with pytest.raises(ValueError):
            op.forward_v3_dp_local_shard(q, k, v, pool[:local_pages].clone(), meta, 0, n_shards)


def test_mla_dp_local_shards_sum_to_the_global_result(gpu):
    """The same scheme for the multi-latent operation over latent pages
    (easydel/operations/kernels/multi_latent_ragged_page_attention.py:507-566)."""
    n_shards, local_pages, page_size, Hq, lkv, rope = 2, 120, 64, 16, 512, 64
    row = orc.mla_page_layout_ref(lkv, rope, page_size)["kv_dim_padded"]
    rng = np.random.default_rng(91)
    S, M = n_shards * 4, 12
    ctx, q_lens, tables = np.zeros(S, np.int32), np.zeros(S, np.int32), np.zeros((S, M), np.int32)
    for sh in range(n_shards):
        free = list(rng.permutation(np.arange(1 if sh == 0 else 0, local_pages)) + sh * local_pages)
        for r, (ql, c) in enumerate([(1, 300), (2, 130), (40, 700)][:3 - sh]):
            i = sh * 4 + r
            ctx[i], q_lens[i] = c + int(rng.integers(0, 60)), ql
            need = -(-int(ctx[i]) // page_size)
            tables[i, :need] = [free.pop() for _ in range(need)]
    qsl = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    T, P = int(qsl[-1]), n_shards * local_pages
    raw = lambda *shape: orc.f32_to_bf16_bits((0.3 * rng.standard_normal(shape)).astype(np.float32))  # noqa: E731
    pages = raw(P, page_size, row)
    qn, qp, kvs, pe = raw(T, Hq, lkv), raw(T, Hq, rope), raw(T, lkv), raw(T, rope)
    up = lambda a: torch.from_numpy(a).to(gpu)  # noqa: E731
    meta = RaggedPagesMetadata(pages_tables=up(tables), context_lens=up(ctx), query_start_loc=up(qsl),
                               num_seqs=torch.tensor([S], dtype=torch.int32, device=gpu),
                               request_distribution=up(orc.request_distribution_ref(q_lens, ctx)), page_size=page_size)
    op = OperationRegistry.create("multi_latent_ragged_page_attention_v1", OperationMetadata())
    pool = tl.to_torch(pages, BF16, gpu)
    scale = (128 + rope) ** -0.5
    outs, new_pages = [], []
    for sh in range(n_shards):
        out, local = op.forward_core_dp_local_shard(tl.to_torch(qn, BF16, gpu), tl.to_torch(qp, BF16, gpu), tl.to_torch(kvs, BF16, gpu),
                                                    tl.to_torch(pe, BF16, gpu), pool[sh * local_pages:(sh + 1) * local_pages].clone(),
                                                    meta, sh, n_shards, softmax_scale=scale)
        torch.cuda.synchronize()
        m = orc.dp_local_shard_ref(sh, n_shards, ctx, tables, qsl, local_pages, T)
        assert not np.abs(tl.from_torch(out, BF16)[~m["token_mask"]]).any(), f"shard {sh}: rows of other ranks' tokens must be zero"
        outs.append(out)
        new_pages.append(local)
    want_pages = orc.mla_page_scatter_ref(kvs, pe, pages, ctx, tables, qsl, [S])
    assert np.array_equal(torch.cat(new_pages).view(torch.int16).cpu().numpy().view(np.uint16), want_pages)
    f = lambda a: orc.bf16_bits_to_f32(a).astype(np.float64)  # noqa: E731
    want = orc.mla_ragged_paged_attention_ref(f(qn), f(qp), f(want_pages), ctx, tables, qsl, [S], kv_lora_rank=lkv, qk_rope_head_dim=rope, softmax_scale=scale)
    err = np.abs(tl.from_torch(dp_local_reduce(outs), BF16) - want)
    assert err.max() <= tl.TOL_BF16_MAX and err.mean() <= tl.TOL_BF16_MEAN, (err.max(), err.mean())


def test_unified_attention_dp_local_shards_sum_to_the_global_result(gpu):
    """The same scheme over separate K and V pools (easydel/operations/kernels/unified_attention.py:278-357); the
    operation only reads the pools."""
    n_shards, local_pages, page_size, Hq, Hkv, D = 2, 300, 64, 32, 8, 128
    b = _sharded_batch(77, n_shards, 5, local_pages, page_size, Hq, Hkv, D)
    up = lambda a: torch.from_numpy(a).to(gpu)  # noqa: E731
    meta = RaggedPagesMetadata(pages_tables=up(b["tables"]), context_lens=up(b["ctx"]), query_start_loc=up(b["qsl"]),
                               num_seqs=torch.tensor([b["S"]], dtype=torch.int32, device=gpu), page_size=page_size)
    q = tl.to_torch(b["q"], BF16, gpu)
    pool = tl.to_torch(b["pages"], BF16, gpu)
    k_pool, v_pool = pool[:, :, 0::2].contiguous(), pool[:, :, 1::2].contiguous()
    op = OperationRegistry.create("unified_attention", OperationMetadata())
    outs = []
    for sh in range(n_shards):
        sl = slice(sh * local_pages, (sh + 1) * local_pages)
        out = op.forward_dp_local_shard(q, k_pool[sl].contiguous(), v_pool[sl].contiguous(), meta, sh, n_shards)
        torch.cuda.synchronize()
        m = orc.dp_local_shard_ref(sh, n_shards, b["ctx"], b["tables"], b["qsl"], local_pages, b["T"])
        assert not np.abs(tl.from_torch(out, BF16)[~m["token_mask"]]).any(), f"shard {sh}: rows of other ranks' tokens must be zero"
        outs.append(out)
    want = orc.ragged_paged_attention_ref(orc.bf16_bits_to_f32(b["q"]).astype(np.float64), orc.bf16_bits_to_f32(b["pages"]).astype(np.float64),
                                          b["ctx"], b["tables"], b["qsl"], [b["S"]])
    err = np.abs(tl.from_torch(dp_local_reduce(outs), BF16) - want)
    assert err.max() <= tl.TOL_BF16_MAX and err.mean() <= tl.TOL_BF16_MEAN, (err.max(), err.mean())
