"""GPU parity of the multi-latent attention entry point on seeded random ragged batches: every seed draws its own head
count, page size and query dtype, a mix of decode, multi-token, chunked-prefill, whole-prompt and empty rows, padding,
and optionally a sliding window, a soft cap, sinks, the read-only call and latent pages of another format than the
queries' (cast-only fp8, float16, bfloat16), and is checked against the float64 oracle
through the C ABI (fused write bit-exact; output to 1e-5 in fp32, 2e-2 max-abs / 5e-3 mean-abs in bf16, one bf16 step where an
output passes |4|)."""

import os

import numpy as np
import pytest

import rpa_testlib as tl
from rpa_testlib import BF16, F16, F32, FP8, make_mla_batch, mla_oracle, run_gpu_mla

pytestmark = pytest.mark.gpu

# (query heads, page size, dtype): bf16 at page sizes of 32 and more runs on the matrix cores, the rest on the fp32 kernel
GEOMETRIES = [(16, 64, BF16), (128, 64, BF16), (20, 32, BF16), (8, 128, BF16), (64, 64, BF16), (5, 16, BF16), (3, 64, F32),
              (1, 64, BF16), (32, 96, BF16)]


# 18 seeds by default; RPA_RANDOM_SEEDS in the environment widens the sweep
_FIRST_SEED = int(os.environ.get("RPA_RANDOM_FIRST_SEED", "0"))  # a sweep over seeds no earlier sweep has seen starts here
# Seeds a wider sweep once failed on, kept as regressions.  758: 20 heads, window 32 -- few visible keys whose values
# cancel; with single bf16 softmax weights in the PV product one output of 3.55 missed by 2.1e-2.
_REGRESSION_SEEDS = [758]
_SEEDS = list(range(_FIRST_SEED, _FIRST_SEED + int(os.environ.get("RPA_RANDOM_SEEDS", "18"))))
_SEEDS += [s for s in _REGRESSION_SEEDS if s not in _SEEDS]


@pytest.mark.parametrize("seed", _SEEDS)
def test_random_mla_batch(gpu, seed):
    rng = np.random.default_rng(5000 + seed)
    Hq, page_size, dtype = GEOMETRIES[seed % len(GEOMETRIES)]
    heavy = Hq >= 64 or dtype == F32  # keeps the float64 oracle within seconds
    n = int(rng.integers(1, 7 if heavy else 12))
    kinds = rng.integers(0, 5, size=n)  # 0 decode, 1 a few tokens, 2 chunk deep in a context, 3 whole prompt, 4 no tokens
    ctx, q_lens = [], []
    for k in kinds:
        if k == 0:
            c = int(rng.integers(1, 1200 if heavy else 3000)); q = 1
        elif k == 1:
            c = int(rng.integers(2, 1000 if heavy else 2500)); q = int(rng.integers(2, min(c, 9) + 1))
        elif k == 2:
            c = int(rng.integers(50, 900 if heavy else 2500)); q = int(rng.integers(10, min(c, 60 if heavy else 200) + 1))
        elif k == 3:
            c = int(rng.integers(1, 100 if heavy else 300)); q = c
        else:
            c = int(rng.integers(0, 500)); q = 0
        ctx.append(c); q_lens.append(q)
    if sum(q_lens) == 0:
        q_lens[0], ctx[0] = 1, max(ctx[0], 1)
    # a generator of its own, so that a seed keeps the batch it always had: one seed in four holds its latent rows in
    # another format (these run on the fp32 kernel, like every page format but the bf16 queries' own)
    fmt = np.random.default_rng(7000 + seed)
    kv_dtype = None
    if Hq <= 32 and fmt.random() < 0.25:
        dtype, kv_dtype = [(BF16, FP8), (F32, FP8), (F16, F16), (F16, FP8), (BF16, F16), (F16, BF16)][int(fmt.integers(0, 6))]
    b = make_mla_batch(6000 + seed, ctx, q_lens, Hq=Hq, page_size=page_size, dtype=dtype, kv_dtype=kv_dtype,
                       pad_rows=int(rng.integers(0, 4)), pad_tokens=int(rng.integers(0, 6)), max_pages=-(-3000 // page_size))
    kw = {"softmax_scale": (128 + 64) ** -0.5}
    if rng.random() < 0.4:
        kw["sliding_window"] = int(rng.integers(1, 600))
    if rng.random() < 0.3:
        kw["logits_soft_cap"] = float(rng.uniform(2.0, 30.0))
    if rng.random() < 0.3:
        kw["softmax_scale"] = float(rng.uniform(0.5, 1.5)) * (128 + 64) ** -0.5
    aux = rng.uniform(-3.0, 7.0, size=Hq).astype(np.float32) if rng.random() < 0.4 else None
    fused = bool(rng.random() < 0.75)
    what = f"seed {seed}: Hq{Hq} pg{page_size} dtype{dtype} pages{kv_dtype} ctx {ctx} q {q_lens} fused={fused} sinks={aux is not None} {sorted(kw)}"
    print(what, flush=True)
    want, want_pages = mla_oracle(b, fused=fused, softmax_aux=aux, **kw)
    got, got_pages = run_gpu_mla(b, fused=fused, softmax_aux=aux, **kw)
    np.testing.assert_array_equal(got_pages, want_pages, err_msg=f"{what}: pages after the call")
    tl.assert_close(got, want, b, what, one_ulp_above_4=True)
    if tl.last_widened:
        print(f"  {tl.last_widened} element(s) with |want| >= 4 judged by one bf16 step instead of 2e-2", flush=True)
    assert np.all(got[int(b.query_start_loc[b.n]):] == 0.0), "padded token rows must be written as zeros"
