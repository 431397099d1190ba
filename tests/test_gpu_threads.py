"""The library from several host threads at once: every thread on a stream and a workspace of its own, the test knobs
belonging to the thread that set them.  Results must be the bits a lone thread gets."""

import threading

import numpy as np
import pytest
import torch

import rpa_testlib as tl
from easydel_amd import _lib, kernels
from rpa_testlib import BF16, FP8

pytestmark = pytest.mark.gpu


def _call(d, b):
    return kernels.ragged_paged_attention(d["query"], d["kv_pages"], d["context_lens"], d["block_tables"], d["query_start_loc"],
                                          d["num_seqs"], kv_scales=d["kv_scales"], num_kv_heads=b.Hkv)


def test_two_threads_two_streams_knobs_stay_with_their_thread(gpu):
    b1 = tl.make_batch(1401, [700, 65, 1500, 300, 33, 2100], [1, 1, 2, 150, 33, 1], Hq=32, Hkv=8, D=128, page_size=64, kv_dtype=BF16)
    b2 = tl.make_batch(1402, [900, 4000, 64, 129, 2500], [1, 3, 1, 129, 300], Hq=40, Hkv=8, D=128, page_size=64, kv_dtype=FP8)
    d1, d2 = tl.device_batch(b1, gpu), tl.device_batch(b2, gpu)
    want1_mfma = _call(d1, b1).clone()
    want2 = _call(d2, b2).clone()
    prev = _lib.set_tunable("force_generic", 1)
    try:
        want1_fp32 = _call(d1, b1).clone()
    finally:
        _lib.set_tunable("force_generic", prev)
    torch.cuda.synchronize()
    assert not torch.equal(want1_fp32, want1_mfma), "the knob must change which kernel runs"
    errors = []
    start = threading.Barrier(2)

    def worker(d, b, want, knob):
        try:
            stream = torch.cuda.Stream(device=gpu)
            with torch.cuda.stream(stream):
                if knob:
                    assert _lib.set_tunable("force_generic", 1) == 0, "a new thread starts from the defaults"
                start.wait(timeout=60)
                for it in range(40):
                    out = _call(d, b)
                    stream.synchronize()
                    if not torch.equal(out, want):
                        errors.append(f"thread knob={knob}: iteration {it} differs from the lone-thread result")
                        return
        except Exception as e:  # noqa: BLE001 - reported to the main thread
            errors.append(f"thread knob={knob}: {type(e).__name__}: {e}")

    threads = [threading.Thread(target=worker, args=(d1, b1, want1_fp32, True)),
               threading.Thread(target=worker, args=(d2, b2, want2, False))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=300)
    assert not any(t.is_alive() for t in threads), "a worker thread did not finish"
    assert not errors, errors
    # the main thread's knobs were never touched by the workers
    assert _lib.set_tunable("force_generic", 0) == 0
    assert torch.equal(_call(d1, b1), want1_mfma)
