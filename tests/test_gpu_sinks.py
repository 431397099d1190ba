"""GPU parity of attention sinks (``softmax_aux``): every kernel that finishes a softmax row -- the decode kernel
(rows it completes alone), the merge kernel (rows split over key spans or key chunks), both prefill kernels and
the fp32 kernel -- against the float64 oracle, through the C ABI."""

import numpy as np
import pytest

import rpa_testlib as tl
from rpa_testlib import BF16, F32, FP8, INT8

pytestmark = pytest.mark.gpu


def _sinks(seed, hq, lo=-2.0, hi=8.0):
    # log-sum-exp of unit-variance scores over a few hundred keys is about 6..8: sinks in this range take anything
    # from a negligible to a dominant share of a row's weight
    return np.random.default_rng(seed).uniform(lo, hi, size=hq).astype(np.float32)


def _check(b, what, sinks, **kw):
    got = tl.run_gpu_attention(b, softmax_aux=sinks, **kw)
    want = tl.oracle_out(b, softmax_aux=sinks, **kw)
    mx, mean = tl.assert_close(got, want, b, what)
    # the case must be able to fail: without the sinks the expected output is far outside the tolerance
    gap = np.abs(tl.oracle_out(b, **kw) - want)[tl.valid_rows(b)].max()
    assert gap > 10 * tl.TOL_BF16_MAX, f"{what}: the sinks change the expected output by only {gap:.2e}"
    print(f"{what}: max-abs {mx:.3e} mean-abs {mean:.3e} (sink effect {gap:.2e})", flush=True)
    return got


@pytest.mark.parametrize("D,page_size,Hq,Hkv,kv_dtype", [(128, 64, 32, 8, BF16), (64, 16, 8, 2, BF16), (256, 128, 16, 8, BF16),
                                                          (64, 32, 64, 8, BF16), (128, 64, 40, 8, FP8), (128, 32, 8, 8, INT8)])
def test_decode_rows_with_sinks(gpu, D, page_size, Hq, Hkv, kv_dtype):
    # short contexts are finished by one workgroup, long ones are cut into spans and merged
    ctx = [1, 2, 17, 64, 65, 300, 1000, 1999, 5000, 128]
    b = tl.make_batch(60 + D, ctx, [1] * len(ctx), Hq=Hq, Hkv=Hkv, D=D, page_size=page_size, kv_dtype=kv_dtype,
                      max_pages=-(-5000 // page_size))
    _check(b, f"decode + sinks D{D} pg{page_size} {Hq}/{Hkv} kv{kv_dtype}", _sinks(D, Hq))


def test_decode_sinks_with_window_and_small_multi_token_rows(gpu):
    ctx = [5, 64, 300, 1100, 777, 4, 2, 3000]
    q_lens = [4, 2, 3, 4, 1, 4, 2, 1]
    b = tl.make_batch(61, ctx, q_lens, Hq=32, Hkv=8, D=128, page_size=64, max_pages=48)
    s = _sinks(61, 32, -1.0, 6.0)
    _check(b, "multi-token small rows + sinks", s)
    _check(b, "multi-token small rows + sinks + window 128", s, sliding_window=128)


@pytest.mark.parametrize("wgs,splits", [(1, 2), (7, 5), (1000, 64)])
def test_sinks_do_not_depend_on_where_sequences_are_cut(gpu, wgs, splits):
    # the sink must enter a row's denominator exactly once however many partial slots the row was split into
    from easydel_amd import _lib

    ctx = [1, 63, 64, 65, 1000, 1999, 128]
    b = tl.make_batch(62, ctx, [1] * len(ctx), Hq=32, Hkv=8, D=128, page_size=64, max_pages=32)
    p1, p2 = _lib.set_tunable("decode_wgs", wgs), _lib.set_tunable("max_splits", splits)
    try:
        _check(b, f"sinks, wgs {wgs} splits {splits}", _sinks(62, 32))
    finally:
        _lib.set_tunable("decode_wgs", p1)
        _lib.set_tunable("max_splits", p2)


@pytest.mark.parametrize("D,page_size,Hq,Hkv,kv_dtype", [(128, 64, 32, 8, BF16), (64, 32, 64, 8, BF16), (256, 128, 16, 8, BF16),
                                                          (128, 16, 40, 8, BF16), (128, 64, 40, 8, FP8), (64, 16, 4, 2, INT8)])
def test_prefill_rows_with_sinks(gpu, D, page_size, Hq, Hkv, kv_dtype):
    # GPT-OSS itself is D 64, 64 query heads over 8 KV heads; page size 16 and 8-bit pages take the register-staged kernel
    ctx = [300, 1000, 129, 47, 2100, 700]
    q_lens = [300, 200, 129, 33, 17, 1]
    b = tl.make_batch(63 + D, ctx, q_lens, Hq=Hq, Hkv=Hkv, D=D, page_size=page_size, kv_dtype=kv_dtype, pad_rows=2, pad_tokens=5)
    s = _sinks(D + 1, Hq)
    got = _check(b, f"prefill + sinks D{D} pg{page_size} {Hq}/{Hkv} kv{kv_dtype}", s)
    assert np.all(got[int(b.query_start_loc[b.n]):] == 0.0)
    _check(b, f"prefill + sinks + window 128 D{D}", s, sliding_window=128)


def test_prefill_sinks_when_row_tiles_are_split_over_key_chunks(gpu):
    # few row tiles over a long prior context: the prefill kernel cuts the keys into chunks and the merge kernel
    # finishes the rows, so that is where the sink joins
    from easydel_amd import _lib

    b = tl.make_batch(64, [40000, 20000], [96, 64], Hq=16, Hkv=4, D=128, page_size=64)
    # over tens of thousands of keys the output of random values averages out to almost nothing; values around one
    # keep it of order one, so that a wrong denominator shows
    vals = b.kv_val.astype(np.float32)
    vals[:, :, 1::2] += 1.0
    b.kv_raw = tl.orc.f32_to_bf16_bits(vals)
    b.kv_val = tl.orc.bf16_bits_to_f32(b.kv_raw).astype(np.float64)
    s = _sinks(64, 16, 8.0, 13.0)  # the log-sum-exp of these rows is about 11
    _check(b, "chunked-key prefill + sinks", s)
    prev = _lib.set_tunable("prefill_chunks", 1)
    try:
        _check(b, "single-chunk prefill + sinks", s)
    finally:
        _lib.set_tunable("prefill_chunks", prev)


def test_fp32_kernel_with_sinks(gpu):
    b = tl.make_batch(65, [17, 64, 130, 255], [1, 1, 8, 33], Hq=8, Hkv=2, D=64, page_size=16, num_pages=128, q_dtype=F32, kv_dtype=F32)
    s = _sinks(65, 8, 0.0, 6.0)
    got = tl.run_gpu_attention(b, softmax_aux=s, softmax_scale=0.125)
    tl.assert_close(got, tl.oracle_out(b, softmax_aux=s, softmax_scale=0.125), b, "fp32 + sinks")  # 1e-5
    got = tl.run_gpu_attention(b, softmax_aux=s, logits_soft_cap=5.0, sliding_window=40)
    tl.assert_close(got, tl.oracle_out(b, softmax_aux=s, logits_soft_cap=5.0, sliding_window=40), b, "fp32 + sinks + cap + window")


def test_soft_cap_does_not_touch_the_sink(gpu):
    b = tl.make_batch(66, [900, 2500, 700], [256, 200, 1], Hq=16, Hkv=8, D=256, page_size=128, max_pages=20)
    _check(b, "soft cap + sinks", _sinks(66, 16, 2.0, 9.0), logits_soft_cap=50.0, softmax_scale=1.0 / 16.0)


def test_infinitely_low_sink_is_bit_identical_to_no_sink_and_huge_sink_gives_zero(gpu):
    ctx = [1500, 900, 300, 40, 2048]
    q_lens = [1, 1, 256, 40, 130]
    b = tl.make_batch(67, ctx, q_lens, Hq=32, Hkv=8, D=128, page_size=64, max_pages=32)
    plain = tl.run_gpu_attention(b)
    low = tl.run_gpu_attention(b, softmax_aux=np.full(32, -np.inf, dtype=np.float32))
    assert np.array_equal(plain, low)
    high = tl.run_gpu_attention(b, softmax_aux=np.full(32, 1e4, dtype=np.float32))
    assert np.all(high == 0.0)


def test_unified_layout_with_sinks(gpu):
    ctx = [17, 64, 130, 255, 500, 33, 1, 3000]
    q_lens = [1, 1, 8, 33, 100, 33, 1, 1]
    b = tl.make_batch(68, ctx, q_lens, Hq=32, Hkv=8, D=64, page_size=32)
    s = _sinks(68, 32)
    got = tl.run_gpu_unified_attention(b, softmax_aux=s, sliding_window=128)
    tl.assert_close(got, tl.oracle_out(b, softmax_aux=s, sliding_window=128), b, "unified + sinks")
    assert np.array_equal(got, tl.run_gpu_attention(b, softmax_aux=s, sliding_window=128))


def test_operations_take_softmax_aux(gpu):
    # through the registry classes, as the reference's GPT-OSS attention layer calls them: the model's per-head
    # sink parameter in the model dtype, GPT-OSS geometry (D 64, 64 query heads over 8 KV heads, window 128)
    import torch

    from easydel_amd.caching import RaggedPagesCacheConfig, RaggedPagesCacheView, RaggedPagesMetadata
    from easydel_amd.operations import OperationMetadata, OperationRegistry

    b = tl.make_batch(69, [200, 64, 700, 2000], [200, 1, 30, 1], Hq=64, Hkv=8, D=64, page_size=32, pad_rows=1)
    d = tl.device_batch(b, gpu)
    s_bf16 = torch.from_numpy(_sinks(69, 64)).to(gpu).to(torch.bfloat16)
    want = tl.oracle_out(b, softmax_aux=s_bf16.float().cpu().numpy(), sliding_window=128)
    cfg = RaggedPagesCacheConfig.create(torch.bfloat16, num_hidden_layers=1, num_kv_heads=8, max_model_length=b.M * 32,
                                        kv_head_dim_size=64, page_size=32, num_pages=b.P)
    view = RaggedPagesCacheView.init(cfg, device=gpu)
    view.kv_pages.copy_(d["kv_pages"].view(view.kv_pages.shape))
    dist = torch.tensor([2, 4, 4], dtype=torch.int32, device=gpu)
    meta = RaggedPagesMetadata(pages_tables=d["block_tables"], context_lens=d["context_lens"], query_start_loc=d["query_start_loc"],
                               num_seqs=d["num_seqs"], request_distribution=dist, page_size=32)
    v2 = OperationRegistry.create("ragged_page_attention_v2", OperationMetadata())
    out = v2(d["query"][None], None, None, view, meta, sliding_window=128, softmax_aux=s_bf16)
    torch.cuda.synchronize()
    assert tuple(out.attention_outputs.shape) == (1, b.T, 64, 64)
    tl.assert_close(tl.from_torch(out.attention_outputs[0], BF16), want, b, "v2 operation + sinks")
    # v3 writes the new tokens' K/V (here: the values the pages already hold at those positions) and attends
    n_valid = int(b.query_start_loc[b.n])
    key = torch.zeros((b.T, 8, 64), dtype=torch.bfloat16, device=gpu)
    value = torch.zeros_like(key)
    pages4 = d["kv_pages"].view(b.P, 32, 16, 64)
    for i in range(b.n):
        for r in range(int(b.q_lens[i])):
            pos = int(b.context_lens[i]) - int(b.q_lens[i]) + r
            row = pages4[int(b.block_tables[i, pos // 32]), pos % 32]
            key[int(b.query_start_loc[i]) + r], value[int(b.query_start_loc[i]) + r] = row[0::2], row[1::2]
    v3 = OperationRegistry.create("ragged_page_attention_v3", OperationMetadata())
    out3 = v3(d["query"], key, value, view, meta, sliding_window=128, softmax_aux=s_bf16)
    torch.cuda.synchronize()
    assert torch.equal(out3.attention_outputs[:n_valid], out.attention_outputs[0, :n_valid])
    with pytest.raises(NotImplementedError, match="one sink logit per query head"):
        v2(d["query"], None, None, view, meta, softmax_aux=torch.zeros(4, 2, device=gpu))
