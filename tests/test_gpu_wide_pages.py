"""GPU parity of the prefill path that serves scaled 8-bit pages through bf16 copies: the decision kernel finds that a
batch's large-row sequences fit the workspace and have rows enough to pay for the copies, their pages are widened once
(bare codes, exact in bf16) and the 32x32-tile kernel reads the copies, scaling each tile's scores by its page's K
scale and its probabilities by the page's V scale.  Checked against the oracle, and against the kernel that reads the 8-bit pages (``prefill_wide`` 0)."""

import os

import numpy as np
import pytest
import torch

import rpa_testlib as tl
from easydel_amd import _lib, kernels
from rpa_testlib import FP8, INT8

pytestmark = pytest.mark.gpu


def _both(b, what, bar=2, **kw):
    """Output with the copies allowed, output with them switched off, both checked against the oracle.  ``bar`` is the
    ``prefill_wide`` knob: 1 the library's rule (1 792 rows per KV head and copied page, or 1 024 in a batch of two
    workgroups per CU), n > 1 a single bar of n rows."""
    want = tl.oracle_out(b, **kw)
    prev = _lib.set_tunable("prefill_wide", bar)
    try:
        got = tl.run_gpu_attention(b, **kw)
    finally:
        _lib.set_tunable("prefill_wide", prev)
    mx, mean = tl.assert_close(got, want, b, what, one_ulp_above_4=True)
    print(f"{what}: max-abs {mx:.3e} mean-abs {mean:.3e}", flush=True)
    prev = _lib.set_tunable("prefill_wide", 0)
    try:
        plain = tl.run_gpu_attention(b, **kw)
    finally:
        _lib.set_tunable("prefill_wide", prev)
    tl.assert_close(plain, want, b, what + " (8-bit kernel)", one_ulp_above_4=True)
    return got, plain


@pytest.mark.parametrize("kv_dtype", [FP8, INT8])
@pytest.mark.parametrize("page_size,Hq,Hkv,D", [(64, 32, 8, 128), (128, 40, 8, 128), (64, 8, 1, 128), (64, 16, 8, 256), (128, 8, 2, 256)])
def test_long_prefill_over_scaled_8bit_pages_reads_the_copies(gpu, kv_dtype, page_size, Hq, Hkv, D):
    """Two long prefill chunks, a short one (large rows too: it is copied with them), decode sequences and an empty row;
    contexts that end inside a page, whose slots past the end hold NaN codes in the fp8 pool."""
    b = tl.make_batch(900 + page_size + Hq, [5000, 1, 700, 9300, 333, 40], [700, 1, 1, 1100, 1, 40], Hq=Hq, Hkv=Hkv, D=D,
                      page_size=page_size, kv_dtype=kv_dtype, pad_rows=2, pad_tokens=5)
    if kv_dtype == FP8:
        for i, c in enumerate(b.context_lens[:b.n]):
            if c % page_size:
                b.kv_raw[b.block_tables[i, c // page_size], c % page_size:] = 0x7F
    got, plain = _both(b, f"copied pages kv{kv_dtype} D{D} pg{page_size} Hq{Hq}/{Hkv}")
    rows = tl.valid_rows(b)
    assert np.abs(got - plain)[rows].max() <= 2 * tl.TOL_BF16_MAX
    assert (got[rows] != plain[rows]).any(), "the two kernels round differently: identical outputs mean the copies were not used"


@pytest.mark.parametrize("kv_dtype", [FP8, INT8])
def test_soft_cap_at_head_size_256_over_the_copies(gpu, kv_dtype):
    """The soft cap's hyperbolic tangent takes the score scaled by the page's K scale (head size 256 only: at 128 the
    32x32-tile kernel has no soft cap)."""
    b = tl.make_batch(920, [4000, 333, 7000, 50], [600, 1, 900, 50], Hq=16, Hkv=8, D=256, page_size=128, kv_dtype=kv_dtype, pad_rows=1)
    for cap in (50.0, 8.0):
        got, plain = _both(b, f"copied pages kv{kv_dtype} D256, soft cap {cap}", logits_soft_cap=cap)
        assert (got[tl.valid_rows(b)] != plain[tl.valid_rows(b)]).any()


def test_key_chunks_over_the_copies(gpu):
    """One prompt chunk behind a long context: its row tiles are cut into key chunks and merged."""
    prev = _lib.set_tunable("prefill_chunks", 8)
    try:
        b = tl.make_batch(911, [30000], [600], Hq=32, Hkv=8, D=128, page_size=64, kv_dtype=INT8)
        got, plain = _both(b, "copied pages, row tiles split over key chunks")
    finally:
        _lib.set_tunable("prefill_chunks", prev)
    b = tl.make_batch(912, [30000, 2000], [600, 300], Hq=32, Hkv=8, D=128, page_size=64, kv_dtype=FP8)
    got, plain = _both(b, "copied pages, chunk length chosen on the device")
    assert (got[tl.valid_rows(b)] != plain[tl.valid_rows(b)]).any()


def test_fp8_pages_without_scales_are_copied_exactly(gpu):
    b = tl.make_batch(913, [4000, 2500], [1200, 400], Hq=32, Hkv=8, D=128, page_size=64, kv_dtype=FP8, scaled=False)
    _both(b, "copied pages, cast-only fp8")


def test_the_librarys_rule_takes_long_chunks(gpu):
    """At the default setting: 4 000 rows per KV head and copied page on average."""
    b = tl.make_batch(917, [4000, 6000, 30], [900, 1300, 1], Hq=32, Hkv=8, D=128, page_size=64, kv_dtype=INT8)
    got, plain = _both(b, "copied pages by the library's rule", bar=1)
    assert (got[tl.valid_rows(b)] != plain[tl.valid_rows(b)]).any()


def test_batches_whose_rows_do_not_pay_stay_on_the_8bit_kernel(gpu):
    """Many short prompt chunks behind long contexts: copying every page would cost more than it saves; the decision
    kernel says no and the result is the 8-bit kernel's, bit for bit -- at a bar of 1 024 rows, and at the library's
    rule for a chunk of 1 200 rows that is far from filling the chip.  Likewise under a soft cap at head size 128, which
    the copies do not serve."""
    b = tl.make_batch(914, [6000] * 8 + [50], [40] * 8 + [1], Hq=32, Hkv=8, D=128, page_size=64, kv_dtype=INT8)
    got, plain = _both(b, "short chunks behind long contexts", bar=1024)
    assert np.array_equal(got, plain)
    b = tl.make_batch(918, [3000, 50], [300, 1], Hq=32, Hkv=8, D=128, page_size=64, kv_dtype=FP8)
    got, plain = _both(b, "one chunk of 1 200 rows", bar=1)
    assert np.array_equal(got, plain)
    b = tl.make_batch(915, [5000, 3000], [700, 600], Hq=32, Hkv=8, D=128, page_size=64, kv_dtype=FP8)
    got, plain = _both(b, "copies not offered with a soft cap at head size 128", logits_soft_cap=30.0)
    assert np.array_equal(got, plain)


@pytest.mark.parametrize("kv_dtype", [FP8, INT8])
@pytest.mark.parametrize("D,page_size,Hq,Hkv,window,cap", [(128, 64, 32, 8, 777, None), (128, 128, 40, 8, 3000, None), (256, 64, 16, 8, 1500, 50.0),
                                                            (128, 64, 8, 1, 64, None)])
def test_sliding_window_over_the_copies(gpu, kv_dtype, D, page_size, Hq, Hkv, window, cap):
    """Under a window only the pages some row of the chunk can see are copied: the first copied page of a sequence is the
    page of its first visible key, wherever that falls inside a page."""
    b = tl.make_batch(930 + window, [5000, 1, 9300, 700, 40], [700, 1, 1100, 300, 40], Hq=Hq, Hkv=Hkv, D=D, page_size=page_size,
                      kv_dtype=kv_dtype, pad_rows=1, pad_tokens=2)
    kw = dict(sliding_window=window)
    if cap:
        kw["logits_soft_cap"] = cap
    got, plain = _both(b, f"copied pages kv{kv_dtype} D{D} pg{page_size} window {window} cap {cap}", **kw)
    assert (got[tl.valid_rows(b)] != plain[tl.valid_rows(b)]).any()


def test_a_workspace_without_room_for_the_copies_falls_back(gpu, monkeypatch):
    """The copies live in what the workspace holds beyond the partial rows: sized without them, the call runs the 8-bit
    kernel (bit-identical to ``prefill_wide`` 0); with room for some pages but not all, likewise."""
    b = tl.make_batch(916, [5000, 700, 9300], [700, 1, 1100], Hq=32, Hkv=8, D=128, page_size=64, kv_dtype=INT8)
    prev = _lib.set_tunable("prefill_wide", 0)
    try:
        plain = tl.run_gpu_attention(b)
        d = tl.device_batch(b)
        lib = _lib.load()
        T, S, M = d["query"].shape[0], b.S, b.M
        small = int(lib.rpa_attention_workspace_bytes(T, S, M, b.page_size, b.Hq, b.Hkv, b.D, tl.BF16, INT8))
    finally:
        _lib.set_tunable("prefill_wide", prev)
    full = int(_lib.load().rpa_attention_workspace_bytes(T, S, M, b.page_size, b.Hq, b.Hkv, b.D, tl.BF16, INT8))
    page16 = b.page_size * 2 * b.Hkv * b.D * 2
    assert full >= small + (79 + 11 + 146) * page16, "the sizing call asks for room for the copies"
    prev = _lib.set_tunable("prefill_wide", 2)
    try:
        for nbytes in (small, small + 100 * page16):
            kernels._workspaces.clear()
            monkeypatch.setattr(kernels, "_workspace", lambda device, n, nb=nbytes: torch.empty(nb, dtype=torch.uint8, device=device))
            got = tl.run_gpu_attention(b)
            assert np.array_equal(got, plain), nbytes
        monkeypatch.undo()
        kernels._workspaces.clear()
        got = tl.run_gpu_attention(b)
    finally:
        _lib.set_tunable("prefill_wide", prev)
    assert (got[tl.valid_rows(b)] != plain[tl.valid_rows(b)]).any()
    tl.assert_close(got, tl.oracle_out(b), b, "full workspace", one_ulp_above_4=True)


@pytest.mark.parametrize("kv_dtype", [FP8, INT8])
def test_separate_key_and_value_pools_are_copied_alike(gpu, kv_dtype):
    """The same through ``unified_attention``: the copy kernel reads K and V rows through the pools' own strides."""
    b = tl.make_batch(919, [3000, 200, 1800], [800, 1, 500], Hq=32, Hkv=8, D=128, page_size=64, kv_dtype=kv_dtype, pad_rows=1)
    want = tl.oracle_out(b)
    prev = _lib.set_tunable("prefill_wide", 2)
    try:
        got = tl.run_gpu_unified_attention(b)
        same = tl.run_gpu_attention(b)
    finally:
        _lib.set_tunable("prefill_wide", prev)
    tl.assert_close(got, want, b, "separate pools, copied pages", one_ulp_above_4=True)
    assert np.array_equal(got, same), "the pool layout changes no bit"
    prev = _lib.set_tunable("prefill_wide", 0)
    try:
        plain = tl.run_gpu_unified_attention(b)
    finally:
        _lib.set_tunable("prefill_wide", prev)
    assert (got[tl.valid_rows(b)] != plain[tl.valid_rows(b)]).any()


@pytest.mark.parametrize("kv_dtype", [FP8, INT8])
def test_fused_quantised_v3_operation_over_long_chunks(gpu, kv_dtype):
    """Registry -> v3 operation on a view with scales, two serving steps with long prompt chunks: the step's K/V rows are
    written quantised first, the copies are made from the pages as written (the rows of this step among them)."""
    from easydel_amd.caching import RaggedPagesCacheConfig, RaggedPagesCacheView, RaggedPagesMetadata
    from easydel_amd.operations import OperationMetadata, OperationRegistry
    from rpa_testlib import BF16, orc

    torch_kv = {FP8: torch.float8_e4m3fn, INT8: torch.int8}[kv_dtype]
    rng = np.random.default_rng(21)
    Hq, Hkv, D, pg, S, M = 32, 8, 128, 64, 4, 40
    P = S * M + 1
    cfg = RaggedPagesCacheConfig.create(torch_kv, num_hidden_layers=1, num_kv_heads=Hkv, max_model_length=M * pg,
                                        kv_head_dim_size=D, page_size=pg, num_pages=P)
    view = RaggedPagesCacheView.init(cfg, device=gpu, scaled=True)
    bt = rng.permutation(np.arange(1, P)).astype(np.int32)[:S * M].reshape(S, M)
    op = OperationRegistry.create("ragged_page_attention_v3", OperationMetadata())
    codes = np.zeros((P, pg, 2 * Hkv, D), np.uint8)
    scales = np.ones((P, 2 * Hkv), np.float32)
    ctx = np.zeros(S, np.int32)
    prev = _lib.set_tunable("prefill_wide", 2)
    try:
        for q_lens in ([1500, 600, 1, 33], [1, 700, 1, 400]):
            q_lens = np.array(q_lens, np.int32)
            ctx = (ctx + q_lens).astype(np.int32)
            qsl = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
            T = int(qsl[-1])
            q_raw, k_raw, v_raw = (orc.f32_to_bf16_bits(rng.standard_normal((T, h, D), dtype=np.float32)) for h in (Hq, Hkv, Hkv))
            dist = orc.request_distribution_ref(q_lens, ctx)
            meta = RaggedPagesMetadata(pages_tables=torch.from_numpy(bt).to(gpu), context_lens=torch.from_numpy(ctx).to(gpu),
                                       query_start_loc=torch.from_numpy(qsl).to(gpu), num_seqs=torch.tensor([S], dtype=torch.int32, device=gpu),
                                       request_distribution=torch.from_numpy(dist).to(gpu), page_size=pg)
            out = op(tl.to_torch(q_raw, BF16, gpu), tl.to_torch(k_raw, BF16, gpu), tl.to_torch(v_raw, BF16, gpu), view, meta)
            torch.cuda.synchronize()
            codes, scales = orc.page_scatter_ragged_quantised_ref(orc.bf16_bits_to_f32(k_raw), orc.bf16_bits_to_f32(v_raw), codes, scales,
                                                                  ctx, bt, qsl, [S], kv_dtype=kv_dtype)
            assert np.array_equal(view.kv_pages.view(torch.uint8).cpu().numpy().reshape(codes.shape), codes)
            assert np.array_equal(view.kv_scales.cpu().numpy(), scales)
            kv_val = orc.decode_codes(codes, kv_dtype).astype(np.float64) * scales[:, None, :, None]
            want = orc.ragged_paged_attention_ref(orc.bf16_bits_to_f32(q_raw).astype(np.float64), kv_val, ctx, bt, qsl, [S])
            got = tl.from_torch(out.attention_outputs, BF16)
            err = np.abs(got - want)
            print(f"  v3 operation over {q_lens.tolist()}: max-abs {err.max():.3e} mean-abs {err.mean():.3e}", flush=True)
            assert err.max() <= tl.TOL_BF16_MAX and err.mean() <= tl.TOL_BF16_MEAN
    finally:
        _lib.set_tunable("prefill_wide", prev)


_SEEDS = int(os.environ.get("RPA_RANDOM_SEEDS", "12"))
_FIRST_SEED = int(os.environ.get("RPA_RANDOM_FIRST_SEED", "0"))


@pytest.mark.parametrize("seed", range(_FIRST_SEED, _FIRST_SEED + _SEEDS))
def test_random_batches_over_the_copies(gpu, seed):
    """Seeded random ragged batches (12 by default, ``RPA_RANDOM_SEEDS`` widens the sweep) with the copies forced: every
    seed draws its heads, page size, page format, a mix of decode rows, short and long chunks, whole prompts and empty
    rows, and optionally sinks and a softmax scale."""
    rng = np.random.default_rng(7000 + seed)
    page_size, Hq, Hkv, D = [(64, 32, 8, 128), (128, 40, 8, 128), (64, 16, 1, 128), (64, 16, 8, 256), (64, 8, 8, 128), (192, 12, 4, 128),
                             (64, 24, 2, 128), (128, 8, 2, 256)][seed % 8]
    kv_dtype, scaled = [(FP8, True), (INT8, True), (FP8, False)][int(rng.integers(0, 3))]
    n = int(rng.integers(1, 9))
    kinds = rng.integers(0, 6, size=n)  # 0 decode, 1 a few tokens, 2 short chunk, 3 long chunk, 4 whole prompt, 5 no tokens
    ctx, q_lens = [], []
    for k in kinds:
        if k == 0:
            c = int(rng.integers(1, 3000)); q = 1
        elif k == 1:
            c = int(rng.integers(2, 2500)); q = int(rng.integers(2, min(c, 12) + 1))
        elif k == 2:
            c = int(rng.integers(50, 5000)); q = int(rng.integers(13, min(c, 200) + 1))
        elif k == 3:
            c = int(rng.integers(300, 6000)); q = int(rng.integers(200, min(c, 1200) + 1))
        elif k == 4:
            c = int(rng.integers(1, 1500)); q = c
        else:
            c = int(rng.integers(0, 500)); q = 0
        ctx.append(c); q_lens.append(q)
    if sum(q_lens) == 0:
        q_lens[0], ctx[0] = 1, max(ctx[0], 1)
    kw = {}
    if rng.random() < 0.3:
        kw["softmax_aux"] = rng.uniform(-3.0, 7.0, size=Hq).astype(np.float32)
    if rng.random() < 0.3:
        kw["softmax_scale"] = float(rng.uniform(0.5, 1.5)) * D ** -0.5
    if D == 256 and rng.random() < 0.5:
        kw["logits_soft_cap"] = float(rng.uniform(5.0, 60.0))
    if rng.random() < 0.35:
        kw["sliding_window"] = int(rng.integers(1, 3000))
    b = tl.make_batch(7100 + seed, ctx, q_lens, Hq=Hq, Hkv=Hkv, D=D, page_size=page_size, kv_dtype=kv_dtype, scaled=scaled,
                      pad_rows=int(rng.integers(0, 3)), pad_tokens=int(rng.integers(0, 6)), shared_prefix_pages=int(rng.integers(0, 3)))
    what = f"seed {seed}: D{D} pg{page_size} {Hq}/{Hkv} kv{kv_dtype}{'' if scaled else ' bare'} ctx {ctx} q {q_lens} {sorted(kw)}"
    print(what, flush=True)
    prev = _lib.set_tunable("prefill_wide", 2)
    try:
        got = tl.run_gpu_attention(b, **kw)
    finally:
        _lib.set_tunable("prefill_wide", prev)
    tl.assert_close(got, tl.oracle_out(b, **kw), b, what, one_ulp_above_4=True)
    assert np.all(got[int(b.query_start_loc[b.n]):] == 0.0), "padded token rows must be written as zeros"


def test_a_call_over_the_copies_replays_from_a_hip_graph(gpu):
    """The decision, the copy and the kernel on the copies are plain launches on the caller's stream: recorded once in a
    graph, every replay gives the eager result, also with the program's own work and synchronisations in between, and
    metadata changed in place (a shorter context) is picked up by the next replay."""
    b = tl.make_batch(950, [4000, 300, 2500], [900, 1, 600], Hq=32, Hkv=8, D=128, page_size=64, kv_dtype=INT8)
    d = tl.device_batch(b)
    out = torch.empty_like(d["query"])

    def call():
        kernels.ragged_paged_attention(d["query"], d["kv_pages"], d["context_lens"], d["block_tables"], d["query_start_loc"], d["num_seqs"],
                                       kv_scales=d["kv_scales"], num_kv_heads=b.Hkv, out=out)

    prev = _lib.set_tunable("prefill_wide", 2)
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            call()  # warm-up on the capture stream: sizes the cached workspace outside the capture
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        eager = out.clone()
        tl.assert_close(tl.from_torch(eager, tl.BF16), tl.oracle_out(b), b, "eager call over the copies", one_ulp_above_4=True)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            call()
        for rep in range(4):
            out.zero_()
            d["query"].mul_(1.0)  # eager work between replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager), f"replay {rep} differs from the eager result"
        d["context_lens"][0] = 3500  # the first chunk now ends 500 tokens earlier: fewer pages to copy, other rows to mask
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        b.context_lens[0] = 3500
        tl.assert_close(tl.from_torch(out, tl.BF16), tl.oracle_out(b), b, "graph replay with new metadata", one_ulp_above_4=True)
    finally:
        _lib.set_tunable("prefill_wide", prev)
