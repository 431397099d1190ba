"""Parity at the benchmark's full sizes: device-generated pools, sampled sequences checked against the
float64 oracle on the pages fetched back, plus size-independent properties."""

import numpy as np
import pytest
import torch

import rpa_testlib as tl
import bench_workloads as workloads
from easydel_amd import kernels
from rpa_testlib import orc

pytestmark = pytest.mark.gpu


def _oracle_on_sample(w, tens, idx, out):
    """Fetch the pages of sequences `idx`, run the oracle on them, compare with the device output rows."""
    worst = 0.0
    for i in idx:
        n_pages = -(-int(w.context_lens[i]) // w.page_size)
        ids = torch.from_numpy(w.block_tables[i, :n_pages].astype(np.int64)).to(out.device)
        pages = tens["kv_pages"][ids]
        scales = None
        if w.kv_dtype == "bf16":
            vals = orc.bf16_bits_to_f32(pages.view(torch.int16).cpu().numpy().view(np.uint16)).astype(np.float64)
        elif w.kv_dtype == "fp8":
            vals = orc.e4m3fn_bits_to_f32(pages.view(torch.uint8).cpu().numpy()).astype(np.float64)
            scales = tens["kv_scales"][ids].cpu().numpy()
        else:
            vals = pages.cpu().numpy().astype(np.float64)
            scales = tens["kv_scales"][ids].cpu().numpy()
        q0, q1 = int(w.query_start_loc[i]), int(w.query_start_loc[i + 1])
        q = orc.bf16_bits_to_f32(tens["query"][q0:q1].view(torch.int16).cpu().numpy().view(np.uint16)).astype(np.float64)
        want = orc.ragged_paged_attention_ref(q, vals, [w.context_lens[i]], np.arange(n_pages)[None], [0, q1 - q0], [1],
                                              softmax_scale=w.softmax_scale, sliding_window=w.sliding_window,
                                              logits_soft_cap=w.logits_soft_cap, kv_scales=scales, num_kv_heads=w.Hkv)
        got = orc.bf16_bits_to_f32(out[q0:q1].view(torch.int16).cpu().numpy().view(np.uint16)).astype(np.float64)
        err = np.abs(got - want)
        assert err.max() <= tl.TOL_BF16_MAX and err.mean() <= tl.TOL_BF16_MEAN, (i, err.max(), err.mean())
        worst = max(worst, err.max())
    return worst


def _oracle_on_rows(w, tens, i, r0, r1, out):
    """Query tokens [r0, r1) of sequence `i` against the oracle, one KV head at a time (a 129 024-token sequence at
    head size 256 is 4 GB in float64 with all heads at once): tokens up to r1 form a chunk that ends at context
    ctx_i - q_len_i + r1, which is what the rows see under the causal rule."""
    q_len, ctx = int(w.q_lens[i]), int(w.context_lens[i])
    ctx_rows = ctx - q_len + r1
    n_pages = -(-ctx_rows // w.page_size)
    ids = torch.from_numpy(w.block_tables[i, :n_pages].astype(np.int64)).to(out.device)
    q0 = int(w.query_start_loc[i])
    G = w.Hq // w.Hkv
    bf = lambda t: orc.bf16_bits_to_f32(t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)).astype(np.float64)  # noqa: E731
    q, got = bf(tens["query"][q0 + r0:q0 + r1]), bf(out[q0 + r0:q0 + r1])
    worst = 0.0
    for h in range(w.Hkv):
        vals = bf(tens["kv_pages"][ids][:, :, 2 * h:2 * h + 2])  # [n_pages, pg, 2, D]: K_h, V_h
        want = orc.ragged_paged_attention_ref(q[:, h * G:(h + 1) * G], vals, [ctx_rows], np.arange(n_pages)[None], [0, r1 - r0], [1],
                                              softmax_scale=w.softmax_scale, sliding_window=w.sliding_window,
                                              logits_soft_cap=w.logits_soft_cap, num_kv_heads=1)
        err = np.abs(got[:, h * G:(h + 1) * G] - want)
        assert err.max() <= tl.TOL_BF16_MAX and err.mean() <= tl.TOL_BF16_MEAN, (i, h, err.max(), err.mean())
        worst = max(worst, err.max())
    return worst


def test_config2_full_size_decode(gpu):
    w = workloads.config2_llama_decode(seed=0)
    assert w.S == 256 and w.num_pages == 40_000 and w.context_lens.min() >= 512 and w.context_lens.max() <= 8192
    tens = workloads.device_tensors(w, gpu, seed=0)
    pool_before = tens["kv_pages"][torch.from_numpy(w.block_tables[:, 0].astype(np.int64)).to(gpu)].clone()
    out, pages = kernels.ragged_paged_attention_v3(tens["query"], tens["key"], tens["value"], tens["kv_pages"], tens["context_lens"],
                                                   tens["block_tables"].reshape(-1), tens["query_start_loc"], tens["distribution"],
                                                   softmax_scale=w.softmax_scale)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    # scatter: each sequence's new token sits bit-exactly at slot (ctx-1) of its last page, and nothing else moved
    view = pages.view(w.num_pages, w.page_size, 2 * w.Hkv, w.D)
    for i in (0, 17, 101, 255):
        pos = int(w.context_lens[i]) - 1
        row = view[int(w.block_tables[i, pos // w.page_size]), pos % w.page_size]
        assert torch.equal(row[0::2], tens["key"][i]) and torch.equal(row[1::2], tens["value"][i])
    first_pages = view[torch.from_numpy(w.block_tables[:, 0].astype(np.int64)).to(gpu)]
    untouched = torch.from_numpy((w.context_lens > w.page_size)).to(gpu)
    assert torch.equal(first_pages[untouched], pool_before.view(first_pages.shape)[untouched])
    # attention: shortest, longest and a few other sequences against the oracle
    idx = sorted({int(np.argmin(w.context_lens)), int(np.argmax(w.context_lens)), 3, 100, 200})
    worst = _oracle_on_sample(w, tens, idx, out)
    print(f"C2 full size: worst max-abs on sampled sequences {worst:.3e}", flush=True)
    # determinism: the split of sequences over workgroups does not depend on timing
    out2, _ = kernels.ragged_paged_attention_v3(tens["query"], tens["key"], tens["value"], tens["kv_pages"], tens["context_lens"],
                                                tens["block_tables"].reshape(-1), tens["query_start_loc"], tens["distribution"],
                                                softmax_scale=w.softmax_scale)
    torch.cuda.synchronize()
    assert torch.equal(out, out2)


@pytest.mark.parametrize("kv_dtype", ["fp8", "int8"])
def test_config4_shape_quantised_decode_reduced_pool(gpu, kv_dtype):
    # the Qwen2.5-32B shape (40 query heads, 8 KV heads) at 64 of its 512 sequences
    w = workloads.config4_quantised_decode(seed=1, kv_dtype=kv_dtype, n_seqs=64, num_pages=18_000)
    tens = workloads.device_tensors(w, gpu, seed=1)
    out = kernels.ragged_paged_attention(tens["query"], tens["kv_pages"], tens["context_lens"], tens["block_tables"],
                                         tens["query_start_loc"], tens["num_seqs"], softmax_scale=w.softmax_scale,
                                         kv_scales=tens["kv_scales"], num_kv_heads=w.Hkv)
    torch.cuda.synchronize()
    worst = _oracle_on_sample(w, tens, [0, 5, int(np.argmax(w.context_lens))], out)
    print(f"C4 {kv_dtype}: worst max-abs {worst:.3e}", flush=True)


@pytest.mark.parametrize("kv_dtype", ["fp8", "int8"])
def test_config4_full_size_quantised_write_and_decode(gpu, kv_dtype):
    """The whole Qwen2.5-32B-shaped configuration: 512 sequences of 4096..16384 tokens over a 140 000-page pool of scaled
    8-bit pages (18 GB: page byte offsets pass 2**34), one new token each, through the fused quantising write +
    attention call.  The write bit for bit against the oracle's rule and the output against the oracle on the pages
    fetched back, for sampled sequences; two runs of the attention bit-identical."""
    w = workloads.config4_quantised_decode(seed=0, kv_dtype=kv_dtype)
    assert w.S == 512 and w.T == 512 and w.num_pages == 140_000 and (w.Hq, w.Hkv, w.D) == (40, 8, 128)
    assert w.context_lens.min() >= 4096 and w.context_lens.max() <= 16384
    tens = workloads.device_tensors(w, gpu, seed=0)
    tag = tl.FP8 if kv_dtype == "fp8" else tl.INT8
    sample = sorted({int(np.argmin(w.context_lens)), int(np.argmax(w.context_lens)), 0, 77, 200, 311, 400, 511})
    codes_of = lambda t: t.view(torch.uint8).cpu().numpy() if kv_dtype == "fp8" else t.cpu().numpy().view(np.uint8)  # noqa: E731
    last = {i: int(w.block_tables[i, (int(w.context_lens[i]) - 1) // w.page_size]) for i in sample}
    before = {i: (codes_of(tens["kv_pages"][last[i]]), tens["kv_scales"][last[i]].cpu().numpy()) for i in sample}
    key, value = tens["key"].to(torch.bfloat16), tens["value"].to(torch.bfloat16)
    out, pages, scales = kernels.ragged_paged_attention_v3_quantised(
        tens["query"], key, value, tens["kv_pages"], tens["kv_scales"], tens["context_lens"], tens["block_tables"].reshape(-1),
        tens["query_start_loc"], tens["distribution"], softmax_scale=w.softmax_scale, num_kv_heads=w.Hkv)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    bf = lambda t: orc.bf16_bits_to_f32(t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16))  # noqa: E731
    for i in sample:  # the page each sampled sequence wrote to, as a one-page problem for the oracle
        slot = (int(w.context_lens[i]) - 1) % w.page_size
        want_codes, want_scales = orc.page_scatter_ragged_quantised_ref(
            bf(key[i:i + 1]), bf(value[i:i + 1]), before[i][0][None], before[i][1][None], [slot + 1], np.zeros((1, 1), np.int32), [0, 1], [1],
            kv_dtype=tag)
        assert np.array_equal(codes_of(pages[last[i]]), want_codes[0].view(np.uint8)), f"codes of sequence {i}'s last page"
        assert np.array_equal(scales[last[i]].cpu().numpy(), want_scales[0]), f"scales of sequence {i}'s last page"
    worst = _oracle_on_sample(w, tens, sample, out)
    print(f"C4 {kv_dtype}, 512 sequences, 140 000 pages: worst max-abs on {len(sample)} sampled sequences {worst:.3e}", flush=True)
    again = [kernels.ragged_paged_attention(tens["query"], pages, tens["context_lens"], tens["block_tables"], tens["query_start_loc"],
                                            tens["num_seqs"], softmax_scale=w.softmax_scale, kv_scales=scales, num_kv_heads=w.Hkv)
             for _ in range(2)]
    torch.cuda.synchronize()
    assert torch.equal(again[0], again[1]) and torch.equal(again[0], out)


def test_config3_mixed_full_size(gpu):
    w = workloads.config3_mixed_chunked(seed=0, num_pages=48_000)
    assert w.T == 2112 and list(w.distribution) == [64, 68, 68]
    tens = workloads.device_tensors(w, gpu, seed=0)
    out, _ = kernels.ragged_paged_attention_v3(tens["query"], tens["key"], tens["value"], tens["kv_pages"], tens["context_lens"],
                                               tens["block_tables"].reshape(-1), tens["query_start_loc"], tens["distribution"],
                                               softmax_scale=w.softmax_scale)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    worst = _oracle_on_sample(w, tens, [0, 63, 64, 67], out)
    print(f"C3: worst max-abs {worst:.3e}", flush=True)


@pytest.mark.parametrize("windowed", [True, False])
def test_config5_gemma_long_context_first_sequence(gpu, windowed):
    # the 63 488-token sequence of the Gemma-2-shaped configuration (soft cap 50, window 4096 or global)
    w = workloads.config5_gemma_long_prefill(seed=0, windowed=windowed)
    tens = workloads.device_tensors(w, gpu, seed=0)
    out = kernels.ragged_paged_attention(tens["query"], tens["kv_pages"], tens["context_lens"], tens["block_tables"],
                                         tens["query_start_loc"], tens["num_seqs"], softmax_scale=w.softmax_scale,
                                         sliding_window=w.sliding_window, logits_soft_cap=w.logits_soft_cap, num_kv_heads=w.Hkv)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    if windowed:
        worst = _oracle_on_sample(w, tens, [0, 1], out)
    else:
        # the global oracle is O(rows * ctx * Hq * D) in float64: slices of rows from the first and the last row tile
        # (a tile is 64 tokens x 2 heads of a group) of both sequences, the 129 024-token one included
        worst = 0.0
        for i, r0, r1 in ((0, 0, 64), (0, 2016, 2048), (1, 0, 32), (1, 1000, 1016), (1, 1984, 2048)):
            e = _oracle_on_rows(w, tens, i, r0, r1, out)
            print(f"  C5 global: sequence {i} (ctx {int(w.context_lens[i])}) tokens [{r0}, {r1}): max-abs {e:.3e}", flush=True)
            worst = max(worst, e)
    print(f"C5 windowed={windowed}: worst max-abs {worst:.3e}", flush=True)


def test_long_context_prefill_over_eight_rounds_of_row_tiles(gpu):
    # 8 sequences of 2 048 prefill tokens at 10k-31k context, Llama-3-8B heads: 256 row tiles of the 32x32 kernel, eight
    # rounds over the chip, every other of which the kernel walks backwards -- a slice of rows from every sequence
    w = workloads.llama_long_prefill(seed=0)
    tens = workloads.device_tensors(w, gpu, seed=0)
    out = kernels.ragged_paged_attention(tens["query"], tens["kv_pages"], tens["context_lens"], tens["block_tables"],
                                         tens["query_start_loc"], tens["num_seqs"], softmax_scale=w.softmax_scale, num_kv_heads=w.Hkv)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    worst = 0.0
    for i in range(len(w.q_lens)):
        r0 = (0, 2032, 992, 64, 1500, 2000, 448, 1216)[i % 8]
        e = _oracle_on_rows(w, tens, i, r0, r0 + 16, out)
        print(f"  long prefill: sequence {i} (ctx {int(w.context_lens[i])}) tokens [{r0}, {r0 + 16}): max-abs {e:.3e}", flush=True)
        worst = max(worst, e)
    print(f"long-context prefill: worst max-abs {worst:.3e}", flush=True)


@pytest.mark.parametrize("kv", ["fp8", "int8"])
def test_quantised_prefill_full_size_reads_the_copies(gpu, kv):
    # 4 x 2 048 prompt tokens behind 8k-16k tokens of scaled 8-bit pages, 40 query heads over 8 KV heads: by the library's
    # own rule the chunks' pages are copied to bf16 once and the 32x32-tile kernel reads the copies; a slice of rows
    # of every sequence against the oracle on the dequantised pages
    from easydel_amd import _lib

    w = workloads.quantised_long_prefill(seed=0, kv_dtype=kv)
    tens = workloads.device_tensors(w, gpu, seed=0)
    att = lambda: kernels.ragged_paged_attention(  # noqa: E731
        tens["query"], tens["kv_pages"], tens["context_lens"], tens["block_tables"], tens["query_start_loc"], tens["num_seqs"],
        softmax_scale=w.softmax_scale, kv_scales=tens["kv_scales"], num_kv_heads=w.Hkv)
    out = att()
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    prev = _lib.set_tunable("prefill_wide", 0)
    try:
        plain = att()
        torch.cuda.synchronize()
    finally:
        _lib.set_tunable("prefill_wide", prev)
    assert not torch.equal(out, plain), "identical bits: the copies were not used"
    assert (out.float() - plain.float()).abs().max().item() <= 2 * tl.TOL_BF16_MAX
    G = w.Hq // w.Hkv
    bf = lambda t: orc.bf16_bits_to_f32(t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)).astype(np.float64)  # noqa: E731
    worst = 0.0
    for i in range(len(w.q_lens)):
        r0 = (0, 2032, 1000, 517)[i % 4]
        r1 = r0 + 16
        ctx_rows = int(w.context_lens[i]) - int(w.q_lens[i]) + r1
        n_pages = -(-ctx_rows // w.page_size)
        ids = torch.from_numpy(w.block_tables[i, :n_pages].astype(np.int64)).to(gpu)
        q0 = int(w.query_start_loc[i])
        q, got = bf(tens["query"][q0 + r0:q0 + r1]), bf(out[q0 + r0:q0 + r1])
        for h in range(w.Hkv):
            vals = (tens["kv_pages"][ids][:, :, 2 * h:2 * h + 2].float() * tens["kv_scales"][ids][:, None, 2 * h:2 * h + 2, None]).double().cpu().numpy()
            want = orc.ragged_paged_attention_ref(q[:, h * G:(h + 1) * G], vals, [ctx_rows], np.arange(n_pages)[None], [0, r1 - r0], [1],
                                                  softmax_scale=w.softmax_scale, num_kv_heads=1)
            err = np.abs(got[:, h * G:(h + 1) * G] - want)
            assert err.max() <= tl.TOL_BF16_MAX and err.mean() <= tl.TOL_BF16_MEAN, (i, h, err.max(), err.mean())
            worst = max(worst, err.max())
    print(f"{kv} prefill through the copies: worst max-abs {worst:.3e}", flush=True)


@pytest.mark.parametrize("Hq", [128, 16])
def test_multi_latent_decode_at_benchmark_size(gpu, Hq):
    """256 sequences of 512..8192 tokens over latent pages (512 + 64, bf16), one new token each: the fused write is in
    place bit-exactly, sampled sequences match the oracle on the pages fetched back, a split over more key chunks
    agrees, and two runs are bit-identical (the unit list is built by scans, not atomics)."""
    from easydel_amd import _lib

    rng = np.random.default_rng(0)
    n, lkv, rope, row, pg = 256, 512, 64, 640, 64
    ctx = rng.integers(512, 8193, size=n).astype(np.int32)
    need = -(-ctx // pg)
    M, P = int(need.max()), int(need.sum()) + 64
    perm = rng.permutation(np.arange(1, P)).astype(np.int32)
    bt = np.zeros((n, M), np.int32)
    k = 0
    for i, m in enumerate(need):
        bt[i, :m] = perm[k:k + m]
        k += m
    g = torch.Generator(device=gpu).manual_seed(1)
    rnd = lambda *shape: torch.randn(*shape, generator=g, device=gpu, dtype=torch.float32).to(torch.bfloat16)  # noqa: E731
    pages = torch.empty(P, pg, row, dtype=torch.bfloat16, device=gpu)
    for lo in range(0, P, 4096):
        pages[lo:lo + 4096] = rnd(min(4096, P - lo), pg, row)
    qn, qp, kv, pe = rnd(n, Hq, lkv), rnd(n, Hq, rope), rnd(n, lkv), rnd(n, rope)
    i32 = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.int32)).to(gpu)  # noqa: E731
    ctx_d, bt_d, qsl_d, dist_d = i32(ctx), i32(bt), i32(np.arange(n + 1)), i32([0, 0, n])
    scale = 192 ** -0.5
    sample = sorted({int(np.argmin(ctx)), int(np.argmax(ctx)), 3, 100, 200})
    last = torch.from_numpy(np.array([bt[i, (ctx[i] - 1) // pg] for i in range(n)], np.int64)).to(gpu)
    before = pages[last].clone()

    out, pages_after = kernels.mla_ragged_paged_attention(qn, qp, kv, pe, pages, ctx_d, bt_d, qsl_d, dist_d, softmax_scale=scale)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    # the write: latent row, rope key, zeroed padding at slot (ctx - 1) of the last page; the other slots untouched
    after = pages_after[last]
    slots = torch.from_numpy(((ctx - 1) % pg).astype(np.int64)).to(gpu)
    rows = after[torch.arange(n, device=gpu), slots]
    assert torch.equal(rows[:, :lkv], kv) and torch.equal(rows[:, lkv:lkv + rope], pe) and not rows[:, lkv + rope:].any()
    keep = torch.ones(n, pg, dtype=torch.bool, device=gpu)
    keep[torch.arange(n, device=gpu), slots] = False
    assert torch.equal(after[keep], before[keep])
    # sampled sequences against the oracle, on the pages as they are now
    bf = lambda t: orc.bf16_bits_to_f32(t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)).astype(np.float64)  # noqa: E731
    worst = 0.0
    for i in sample:
        m = int(need[i])
        seq_pages = bf(pages_after[torch.from_numpy(bt[i, :m].astype(np.int64)).to(gpu)])
        want = orc.mla_ragged_paged_attention_ref(bf(qn[i:i + 1]), bf(qp[i:i + 1]), seq_pages, [ctx[i]], np.arange(m)[None], [0, 1], [1],
                                                  kv_lora_rank=lkv, qk_rope_head_dim=rope, softmax_scale=scale)
        err = np.abs(bf(out[i:i + 1]) - want)
        assert err.max() <= tl.TOL_BF16_MAX and err.mean() <= tl.TOL_BF16_MEAN, (i, err.max(), err.mean())
        worst = max(worst, err.max())
    print(f"MLA decode, {Hq} heads, full size: worst max-abs on sampled sequences {worst:.3e}", flush=True)
    # read-only repeats: bit-identical run to run; more key chunks: the same within the tolerance
    again, _ = kernels.mla_ragged_paged_attention(qn, qp, None, None, pages_after, ctx_d, bt_d, qsl_d, dist_d, softmax_scale=scale)
    again2, _ = kernels.mla_ragged_paged_attention(qn, qp, None, None, pages_after, ctx_d, bt_d, qsl_d, dist_d, softmax_scale=scale)
    torch.cuda.synchronize()
    assert torch.equal(again, again2) and torch.equal(again, out)
    prev = _lib.set_tunable("mla_chunks", 8)
    try:
        split, _ = kernels.mla_ragged_paged_attention(qn, qp, None, None, pages_after, ctx_d, bt_d, qsl_d, dist_d, softmax_scale=scale)
        torch.cuda.synchronize()
    finally:
        _lib.set_tunable("mla_chunks", prev)
    assert (split.float() - out.float()).abs().max().item() <= tl.TOL_BF16_MAX


def test_pages_at_the_top_of_a_160_gib_pool(gpu):
    """The pool a 288 GB card can hold: page byte offsets beyond 2**37.  A mixed batch whose pages all lie in the last
    few hundred pages of a 160 GiB pool (the rest is never initialised and never read) goes through the fused write +
    attention call: the written pages bit-exact, the output against the oracle, and the same bits as the same batch in
    a small pool."""
    Hq, Hkv, D, pg = 32, 8, 128, 64
    b = tl.make_batch(91, [700, 65, 1500, 300, 2000, 4100], [1, 1, 2, 300, 1, 40], Hq=Hq, Hkv=Hkv, D=D, page_size=pg, pad_rows=2)
    rng = np.random.default_rng(92)
    key_raw = orc.f32_to_bf16_bits(rng.standard_normal((b.T, Hkv, D), dtype=np.float32))
    val_raw = orc.f32_to_bf16_bits(rng.standard_normal((b.T, Hkv, D), dtype=np.float32))
    key_val = orc.bf16_bits_to_f32(key_raw).astype(np.float64)
    val_val = orc.bf16_bits_to_f32(val_raw).astype(np.float64)
    want_pages = orc.page_scatter_ragged_ref(key_val, val_val, b.kv_val, b.context_lens, b.block_tables, b.query_start_loc, b.num_seqs)
    want = tl.oracle_out(b, kv_val=want_pages)

    page_bytes = pg * 2 * Hkv * D * 2
    P_big = (160 << 30) // page_bytes
    base = P_big - b.P
    assert base * page_bytes > (1 << 37)
    torch.cuda.empty_cache()  # a pool an earlier test has dropped still sits in torch's allocator
    free, _ = torch.cuda.mem_get_info()
    if free < (P_big * page_bytes) + (4 << 30):
        pytest.skip(f"needs a 160 GiB pool, {free >> 30} GiB free on this device")
    d = tl.device_batch(b, gpu)
    key, val = tl.to_torch(key_raw, tl.BF16, gpu), tl.to_torch(val_raw, tl.BF16, gpu)
    dist = torch.tensor([0, 0, b.n], dtype=torch.int32, device=gpu)
    print(f"[pool] {P_big} pages of {page_bytes} B, batch pages at {base}..{P_big - 1}", flush=True)

    small = d["kv_pages"].clone()
    out_small, small = kernels.ragged_paged_attention_v3(d["query"], key, val, small, d["context_lens"], d["block_tables"],
                                                         d["query_start_loc"], dist)
    big = torch.empty((P_big, pg, 2 * Hkv, D), dtype=torch.bfloat16, device=gpu)
    big[base:] = d["kv_pages"]
    bt_big = torch.where(d["block_tables"] > 0, d["block_tables"] + base, d["block_tables"])
    out_big, big = kernels.ragged_paged_attention_v3(d["query"], key, val, big, d["context_lens"], bt_big, d["query_start_loc"], dist)
    torch.cuda.synchronize()
    got_pages = tl.from_torch(big[base:], tl.BF16)
    np.testing.assert_array_equal(got_pages, want_pages, err_msg="pages after the write at the top of the pool")
    tl.assert_close(tl.from_torch(out_big, tl.BF16), want, b, "160 GiB pool")
    assert torch.equal(out_big, out_small), "the same batch must give the same bits wherever its pages lie"
    del big
    torch.cuda.empty_cache()


def test_latent_pages_at_the_top_of_a_160_gib_pool(gpu):
    """The same for the multi-latent call: latent pages (80 KiB each) at the top of a 160 GiB pool."""
    b = tl.make_mla_batch(93, [700, 65, 1500, 300, 2000], [1, 1, 2, 150, 1], Hq=16, pad_rows=1)
    want, want_pages = tl.mla_oracle(b, fused=True, softmax_scale=(128 + 64) ** -0.5)
    page_bytes = b.page_size * b.row * 2
    P_big = (160 << 30) // page_bytes
    base = P_big - b.P
    torch.cuda.empty_cache()  # a pool an earlier test has dropped still sits in torch's allocator
    free, _ = torch.cuda.mem_get_info()
    if free < (P_big * page_bytes) + (4 << 30):
        pytest.skip(f"needs a 160 GiB pool, {free >> 30} GiB free on this device")
    t = lambda raw: tl.to_torch(raw, tl.BF16, gpu)
    i32 = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.int32)).to(gpu)
    big = torch.empty((P_big, b.page_size, b.row), dtype=torch.bfloat16, device=gpu)
    big[base:] = t(b.pages_raw)
    bt_big = np.where(b.block_tables > 0, b.block_tables + base, b.block_tables)
    print(f"[pool] {P_big} latent pages of {page_bytes} B, batch pages at {base}..{P_big - 1}", flush=True)
    out, big = kernels.mla_ragged_paged_attention(t(b.qn_raw), t(b.qp_raw), t(b.kv_raw), t(b.pe_raw), big, i32(b.context_lens),
                                                  i32(bt_big), i32(b.query_start_loc), i32(b.distribution),
                                                  softmax_scale=(128 + 64) ** -0.5)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(tl.from_torch(big[base:], tl.BF16), want_pages, err_msg="latent pages after the write")
    tl.assert_close(tl.from_torch(out, tl.BF16), want, b, "160 GiB latent pool")
    del big
    torch.cuda.empty_cache()
