"""Parity of the multi-latent attention entry point (rpa_mla_ragged_paged_attention, through the C ABI) against the
numpy oracle: the fused write bit-exact, the attention output to 1e-5 (fp32) / 2e-2 max-abs, 5e-3 mean-abs (bf16)."""

import numpy as np
import pytest

import rpa_testlib as tl
from rpa_testlib import BF16, F16, F32, FP8, orc

pytestmark = pytest.mark.gpu


from rpa_testlib import make_mla_batch, mla_oracle, run_gpu_mla  # noqa: E402


def check(b, what, *, fused=True, softmax_aux=None, **kw):
    print(f"[mla] {what}: T={b.T} S={b.S} Hq={b.Hq} lkv={b.lkv} rope={b.rope} pg={b.page_size} kw={kw}", flush=True)
    want, want_pages = mla_oracle(b, fused=fused, softmax_aux=softmax_aux, **kw)
    got, got_pages = run_gpu_mla(b, fused=fused, softmax_aux=softmax_aux, **kw)
    np.testing.assert_array_equal(got_pages, want_pages, err_msg=f"{what}: pages after the write")
    # latent rows are N(0,1) in 512 dims and a row with one dominant key returns them: outputs beyond 4 do occur here
    r = tl.assert_close(got, want, b, what, one_ulp_above_4=True)
    if tl.last_widened:
        print(f"  {tl.last_widened} element(s) with |want| >= 4 judged by one bf16 step instead of 2e-2", flush=True)
    return r


SCALE = (128 + 64) ** -0.5  # what the caller passes for DeepSeek-V3: (qk_nope_head_dim + qk_rope_head_dim) ** -0.5


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_small_shapes_run_on_the_fp32_kernel(dtype):
    b = make_mla_batch(0, [17, 64, 130, 255, 1], [1, 1, 8, 33, 1], Hq=4, lkv=64, rope=16, page_size=16, dtype=dtype, pad_rows=2, pad_tokens=3)
    check(b, "small", softmax_scale=0.11)
    check(b, "small window+cap", softmax_scale=0.11, sliding_window=20, logits_soft_cap=5.0)
    check(b, "small read-only", fused=False)
    check(b, "small sinks", softmax_aux=np.array([0.5, -1.0, 2.0, 0.0]))


@pytest.mark.parametrize("dtype,kv_dtype", [(BF16, FP8), (F32, FP8), (F16, F16), (F16, FP8), (BF16, F16), (F16, BF16)])
def test_cast_only_fp8_and_float16_latent_pages(dtype, kv_dtype):
    # the reference's latent cache takes any floating kvdtype and holds no scale arrays
    # (caching/mla_ragged_page/cache.py:197-204, 344): fp8 pages are plain casts.  These formats run on the fp32 kernel.
    b = make_mla_batch(11, [17, 64, 130, 255, 1], [1, 1, 8, 33, 1], Hq=4, lkv=64, rope=16, page_size=16, dtype=dtype,
                       kv_dtype=kv_dtype, pad_rows=2, pad_tokens=3)
    check(b, "formats small", softmax_scale=0.11)
    check(b, "formats small window+cap", softmax_scale=0.11, sliding_window=20, logits_soft_cap=5.0)
    check(b, "formats small read-only", fused=False)


@pytest.mark.parametrize("dtype,kv_dtype", [(BF16, FP8), (F16, F16)])
def test_fp8_and_float16_latent_pages_at_the_model_shape(dtype, kv_dtype):
    rng = np.random.default_rng(12)
    ctx = rng.integers(1, 900, size=6).tolist() + [300, 77]
    b = make_mla_batch(13, ctx, [1] * 6 + [40, 77], Hq=16, dtype=dtype, kv_dtype=kv_dtype, pad_rows=1, pad_tokens=2)
    check(b, "formats 512+64", softmax_scale=SCALE)


def test_fp32_queries_at_the_model_shape():
    b = make_mla_batch(1, [70, 300, 5], [1, 4, 5], Hq=3, page_size=32, dtype=F32)
    check(b, "fp32 512+64", softmax_scale=SCALE)


@pytest.mark.parametrize("Hq", [16, 128, 20])
def test_decode_batches_on_the_matrix_cores(Hq):
    rng = np.random.default_rng(2)
    ctx = rng.integers(1, 700, size=9).tolist() + [1, 32, 33, 64, 65]
    b = make_mla_batch(3, ctx, [1] * len(ctx), Hq=Hq, pad_rows=3, pad_tokens=2)
    check(b, f"decode Hq={Hq}", softmax_scale=SCALE)


def test_more_row_tile_slots_than_the_sorted_unit_list_holds():
    # 3 900 single tokens at 8 heads: 4 143 row-tile slots, so a decode batch takes the plan and unit list of large batches
    # (two launches, slot order) instead of the one-block sorted list
    rng = np.random.default_rng(7)
    ctx = rng.integers(1, 33, size=3900).tolist()
    b = make_mla_batch(8, ctx, [1] * len(ctx), Hq=8, page_size=32, pad_rows=10, pad_tokens=2, distinct_pages=97)
    assert b.T * b.Hq // 128 + b.S > 4096
    check(b, "3900 sequences", softmax_scale=SCALE)


def test_unit_list_in_length_classes():
    # 700 sequences at 16 heads: 797 row-tile slots -- more than the exact sort of the unit list takes (512), fewer than
    # the one-block plan holds (4 096): the list is built longest first in eight length classes.  Contexts of 1 ... 2 500
    # keys, so that the long ones are cut into chunks and the classes are all in use.
    rng = np.random.default_rng(21)
    ctx = rng.integers(1, 400, size=700)
    ctx[::37] = rng.integers(1200, 2500, size=len(ctx[::37]))
    b = make_mla_batch(22, ctx.tolist(), [1] * len(ctx), Hq=16, page_size=64, pad_rows=5, pad_tokens=3, distinct_pages=211)
    slots = b.T * b.Hq // 128 + b.S
    assert 512 < slots <= 4096
    check(b, "700 sequences", softmax_scale=SCALE)


def test_chunked_prefill_and_mixed_rows():
    b = make_mla_batch(4, [200, 97, 400, 31, 1000], [1, 97, 150, 31, 3], Hq=16)
    check(b, "mixed", softmax_scale=SCALE)
    b = make_mla_batch(5, [300, 64], [40, 64], Hq=128, page_size=32)
    check(b, "prefill Hq=128 pg=32", softmax_scale=SCALE)


def test_window_soft_cap_and_sinks_on_the_matrix_cores():
    b = make_mla_batch(6, [500, 260, 90, 700], [1, 130, 90, 5], Hq=16)
    check(b, "window", softmax_scale=SCALE, sliding_window=100)
    check(b, "window 1", softmax_scale=SCALE, sliding_window=1)
    check(b, "cap", softmax_scale=SCALE, logits_soft_cap=2.0)
    check(b, "sinks", softmax_scale=SCALE, softmax_aux=np.linspace(-2.0, 3.0, 16))
    check(b, "read-only", softmax_scale=SCALE, fused=False)


def test_rows_split_over_key_chunks_agree_with_single_chunks():
    from easydel_amd import _lib

    b = make_mla_batch(7, [2500, 1300, 700, 4000], [1, 2, 70, 1], Hq=16)
    for chunks in (1, 3, 16):
        prev = _lib.set_tunable("mla_chunks", chunks)
        try:
            check(b, f"chunks={chunks}", softmax_scale=SCALE)
            check(b, f"chunks={chunks} window", softmax_scale=SCALE, sliding_window=1500)
            check(b, f"chunks={chunks} sinks", softmax_scale=SCALE, softmax_aux=np.linspace(-1.0, 4.0, 16))
        finally:
            _lib.set_tunable("mla_chunks", prev)
    check(b, "default chunks", softmax_scale=SCALE)


def test_matrix_core_kernel_matches_the_fp32_kernel():
    from easydel_amd import _lib

    b = make_mla_batch(8, [333, 64, 1200], [1, 64, 20], Hq=32)
    got, _ = run_gpu_mla(b, softmax_scale=SCALE)
    prev = _lib.set_tunable("force_generic", 1)
    try:
        ref, _ = run_gpu_mla(b, softmax_scale=SCALE)
    finally:
        _lib.set_tunable("force_generic", prev)
    rows = tl.valid_rows(b)
    assert np.abs(got[rows] - ref[rows]).max() <= 2e-2


def test_large_scores_raise_the_softmax_reference():
    # scores growing along the sequence (through the rope part, so the values stay of order one) force the running
    # reference up tile after tile
    b = make_mla_batch(9, [600], [1], Hq=16)
    ramp = np.linspace(0.0, 40.0, 600)
    pages = b.pages_val.copy()
    qp = np.zeros_like(b.qp_val); qp[..., 0] = 1.0
    for pos in range(599):
        pages[b.block_tables[0, pos // 64], pos % 64, b.off] = ramp[pos]
    b.pe_val[0, 0] = 40.0
    b.pe_raw = orc.f32_to_bf16_bits(b.pe_val.astype(np.float32)); b.pe_val = orc.bf16_bits_to_f32(b.pe_raw).astype(np.float64)
    b.pages_raw = orc.f32_to_bf16_bits(pages.astype(np.float32)); b.pages_val = orc.bf16_bits_to_f32(b.pages_raw).astype(np.float64)
    b.qp_raw = orc.f32_to_bf16_bits(qp.astype(np.float32)); b.qp_val = orc.bf16_bits_to_f32(b.qp_raw).astype(np.float64)
    b.qn_raw = np.zeros_like(b.qn_raw); b.qn_val = np.zeros_like(b.qn_val)
    check(b, "ramp", softmax_scale=1.0)


def test_padded_tokens_are_zeroed_and_bad_arguments_are_reported():
    import torch

    from easydel_amd import _lib, kernels

    b = make_mla_batch(10, [100, 50], [1, 1], Hq=16, pad_tokens=5)
    got, _ = run_gpu_mla(b, softmax_scale=SCALE)
    assert not got[2:].any()
    q = torch.zeros(2, 16, 512, dtype=torch.bfloat16, device="cuda:0")
    pages = torch.zeros(4, 64, 576 - 8, dtype=torch.bfloat16, device="cuda:0")  # row too short for latent + rope
    i = lambda *v: torch.tensor(v, dtype=torch.int32, device="cuda:0")
    with pytest.raises(_lib.RpaError, match="row_elems"):
        kernels.mla_ragged_paged_attention(q, q[..., :64].contiguous(), None, None, pages, i(5, 5), i(1, 2), i(0, 1, 2), i(0, 0, 2))
    with pytest.raises(ValueError, match="must share"):
        kernels.mla_ragged_paged_attention(q, q[:1, :, :64].contiguous(), None, None, pages, i(5, 5), i(1, 2), i(0, 1, 2), i(0, 0, 2))


def test_hip_graph_replay_matches_eager_and_follows_new_metadata():
    # the call neither allocates nor synchronises nor clears memory with a memset node: the write, the plan, the unit
    # list, the attention (rows split over key chunks) and the merge replay from a captured graph
    import torch

    from easydel_amd import kernels

    dev = "cuda:0"
    b = make_mla_batch(11, [2500, 65, 700, 1, 1200], [1, 1, 30, 1, 2], Hq=16, pad_rows=2, pad_tokens=1)
    t = lambda raw: tl.to_torch(raw, BF16, dev)  # noqa: E731
    i32 = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.int32)).to(dev)  # noqa: E731
    qn, qp, kv, pe, pages = t(b.qn_raw), t(b.qp_raw), t(b.kv_raw), t(b.pe_raw), t(b.pages_raw)
    ctx, bt, qsl, dist = i32(b.context_lens), i32(b.block_tables), i32(b.query_start_loc), i32(b.distribution)
    out = torch.empty_like(qn)

    def call():
        kernels.mla_ragged_paged_attention(qn, qp, kv, pe, pages, ctx, bt, qsl, dist, softmax_scale=SCALE, out=out)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()  # warm-up on the capture stream: sizes the cached workspace outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    eager = out.clone()
    want, _ = mla_oracle(b, softmax_scale=SCALE)
    tl.assert_close(tl.from_torch(eager, BF16), want, b, "eager")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        call()
    for rep in range(4):
        out.zero_()
        qn.mul_(1.0)  # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {rep} differs from the eager result"
    ctx[0] = 2100  # new metadata in the same buffers: nothing is baked in on the host
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    b.context_lens[0] = 2100
    b.pages_raw = pages.view(torch.int16).cpu().numpy().view(np.uint16)  # the pages as the replays left them
    b.pages_val = orc.bf16_bits_to_f32(b.pages_raw).astype(np.float64)
    want, _ = mla_oracle(b, softmax_scale=SCALE)
    tl.assert_close(tl.from_torch(out, BF16), want, b, "graph replay with new metadata")
