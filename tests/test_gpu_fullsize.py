"""Parity at the benchmark's full sizes: device-generated pools, sampled sequences checked against the
float64 oracle on the pages fetched back, plus size-independent properties."""

import numpy as np
import pytest
import torch

import rpa_testlib as tl
from easydel_amd import kernels, workloads
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
    else:  # the global oracle is O(q_len * ctx * Hq * D) in float64: check a slice of rows of sequence 0
        w2 = workloads.Workload(w.name, w.Hq, w.Hkv, w.D, w.page_size, w.num_pages, w.max_pages_per_seq,
                                w.context_lens[:1] - 2048 + 64, np.array([64], np.int32), w.block_tables[:1],
                                softmax_scale=w.softmax_scale, logits_soft_cap=w.logits_soft_cap)
        worst = _oracle_on_sample(w2, tens, [0], out)
    print(f"C5 windowed={windowed}: worst max-abs {worst:.3e}", flush=True)


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
