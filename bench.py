#!/usr/bin/env python3
"""Benchmark of the ragged-paged-attention hot path on one MI355X.

A step is one attention-layer call of the serving path on one ragged batch: the page scatter
that writes the new K/V rows, then the attention over the paged cache (the fused v3 entry
point of the C ABI).  The default workload is the Llama-3-8B-shaped pure decode batch
(256 sequences, 512-8192 tokens of context, bf16, 64-token pages, 40 000-page pool).

Prints one JSON line.  ``value`` = query tokens per second of one layer call with every
input resident in HBM; ``roofline`` describes the dominant kernel (decode attention), timed
with events on the launch stream in isolation; ``cpu_baseline`` times the C restatement of
the same operation (oracle/rpa_oracle_c.c) on the host cores over a bounded sample.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16 MFMA rate


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=25,
                    help="untimed calls ahead of the timed ones (the first twenty or so calls of a workload run a few percent slower than the later ones)")
    ap.add_argument("--workload", default="c2", choices=["c2", "c3", "c4-fp8", "c4-int8", "c5-global", "c5-window", "llama-prefill", "fp8-prefill", "int8-prefill", "int8-prefill-d256", "int8-prefill-d256-cap", "gemma-decode",
                             "decode-hkv4", "decode-hkv1", "decode-16seq", "decode-32seq",
                             "mla-decode-h128", "mla-decode-h16", "mla-prefill-h128"])
    ap.add_argument("--layout", default="interleaved", choices=["interleaved", "unified"],
                    help="interleaved: one pool [P, page, 2*Hkv, D], scatter fused with the attention call (v3); "
                         "unified: separate K and V pools [P, page, Hkv, D], two slice scatters then the attention call")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra-configs", action="store_true",
                    help="default workload only: do not measure the other benchmark configurations afterwards")
    ap.add_argument("--hip-graph", action="store_true",
                    help="also time the step recorded once in a HIP graph and replayed (ms_per_step_hip_graph)")
    ap.add_argument("--mfma-probe", action="store_true",
                    help="instead of a workload: the library's matrix-core feed probe (bf16 MFMA streams with operands from "
                         "registers or LDS, both tile shapes, 1 / 2 / 4 MFMAs per operand, one and two waves per SIMD), one line per setting")
    ap.add_argument("--issue-probe", action="store_true",
                    help="what one more instruction of a kind costs a lone wave per SIMD beside a stream of 32x32x16 MFMAs (rpa_issue_probe)")
    ap.add_argument("--cpu-sample-seqs", type=int, default=0, help="sequences in the CPU sample (0 = auto)")
    ap.add_argument("--decode-wgs", type=int, default=0)
    ap.add_argument("--prefill-chunks", type=int, default=0)
    ap.add_argument("--decode-sync", type=int, default=-1)
    ap.add_argument("--decode-dma", type=int, default=-1, help="LDS-direct decode kernel: -1 the library's choice, 0 never, 1 wherever built")
    ap.add_argument("--max-splits", type=int, default=0)
    ap.add_argument("--prefill-x32", type=int, default=-1, help="32x32-tile prefill kernel: -1 the library's choice, 0 never")
    ap.add_argument("--prefill-wide", type=int, default=-1, help="bf16 copies of 8-bit pages for the 32x32-tile prefill kernel: -1 the library's choice, 0 never")
    ap.add_argument("--chunk-seqs", type=int, default=0, help="fp8-prefill / int8-prefill: this many prompt chunks (1..16) instead of 4 ...")
    ap.add_argument("--chunk-len", type=int, default=0, help="... of this many tokens instead of 2 048")
    ap.add_argument("--chunk-window", type=int, default=0, help="the 8-bit prefill shapes under a sliding window of this many tokens")
    ap.add_argument("--mla-chunks", type=int, default=0)
    ap.add_argument("--mla-min-chunk", type=int, default=0)
    ap.add_argument("--mla-uniform-context", type=int, default=0,
                    help="multi-latent decode workloads: every sequence this long (with --mla-chunks 1: one equal unit of "
                         "work per sequence, which separates the cost of a tile from the cost of a unit and of imbalance)")
    ap.add_argument("--mla-distinct-pages", type=int, default=0,
                    help="multi-latent decode workloads: the block tables name only this many different pages, so that the "
                         "latent rows come out of the L2 instead of HBM (what the kernel costs with memory taken away)")
    ap.add_argument("--sequential-pages", action="store_true", help="experiment: block tables in pool order")
    ap.add_argument("--read-probe", action="store_true",
                    help="instead of a workload: time the library's read-only probe over 8 GiB for 32..256 workgroups and "
                         "16..256 KiB in flight per workgroup, one line per setting")
    ap.add_argument("--read-probe-paged", action="store_true",
                    help="instead of a workload: time the paged read probe (the decode kernel's access pattern without its "
                         "arithmetic: chunk size, split over the waves, load flavour, bytes in flight), one line per setting")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy, so a counter run shows what a known-size kernel reads")
    return ap.parse_args()


DECODE_SHAPES = {"decode-hkv4": dict(Hq=28, Hkv=4), "decode-hkv1": dict(Hq=8, Hkv=1), "decode-16seq": dict(n_seqs=16),
                 "decode-32seq": dict(n_seqs=32)}


def build_workload(name, seed, sequential=False, chunks=(0, 0)):
    import bench_workloads as workloads

    if name == "c2":
        return workloads.config2_llama_decode(seed, shuffle_pages=not sequential)
    if name == "c3":
        return workloads.config3_mixed_chunked(seed)
    if name == "c4-fp8":
        return workloads.config4_quantised_decode(seed, "fp8")
    if name == "c4-int8":
        return workloads.config4_quantised_decode(seed, "int8")
    if name in ("int8-prefill-d256", "int8-prefill-d256-cap"):
        kw = dict(n_seqs=chunks[0], q_len=chunks[1], num_pages=6000 if chunks[0] > 4 else 2000) if chunks[0] > 0 and chunks[1] > 0 else {}
        return workloads.quantised_long_prefill(seed, "int8", head_dim=256, soft_cap=50.0 if name.endswith("-cap") else None, **kw)
    if name in ("fp8-prefill", "int8-prefill"):  # tuning shape for the 8-bit prefill kernel
        if chunks[0] > 0 and chunks[1] > 0:  # (6 000 pages hold 16 chunks of up to 16 384 tokens of context)
            return workloads.quantised_long_prefill(seed, name.split("-")[0], n_seqs=chunks[0], q_len=chunks[1], num_pages=6000 if chunks[0] > 4 else 2000)
        return workloads.quantised_long_prefill(seed, name.split("-")[0])
    if name == "gemma-decode":  # tuning shape: decode at head size 256, where the LDS-direct decode kernel is the default
        return workloads.gemma_decode(seed)
    if name == "llama-prefill":  # tuning shape for the prefill kernel, not one of the benchmark configurations
        return workloads.llama_long_prefill(seed)
    if name in DECODE_SHAPES:  # tuning shapes: decode away from the benchmark's head counts and batch size
        return workloads.decode_shape(seed, **DECODE_SHAPES[name])
    return workloads.config5_gemma_long_prefill(seed, windowed=(name == "c5-window"))


KERNEL_SOURCES = {  # the files a kernel is compiled from: a counter run is only valid for the sources it was taken on
    "attn_decode_kernel": ("rpa_attn_decode.hip", "rpa_attn_decode_dma.h", "rpa_mfma.h", "rpa_common.h"),
    "attn_prefill_kernel": ("rpa_attn_prefill_x32.hip", "rpa_attn_prefill_dma.hip", "rpa_attn_prefill_dma8.hip", "rpa_attn_prefill.hip", "rpa_widen.hip", "rpa_mfma.h", "rpa_common.h"),
}


def kernel_source_sha16(kernel):
    """First 16 hex digits of the SHA-256 over the source files of a kernel (KERNEL_SOURCES), in order."""
    import hashlib

    h = hashlib.sha256()
    for name in KERNEL_SOURCES[kernel]:
        with open(os.path.join(ROOT, "easydel_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(workload, kernel="attn_decode_kernel"):
    """``(bytes, source)``: HBM bytes per launch of a kernel from a committed counter run (FETCH_SIZE and WRITE_SIZE
    passes of rocprofv3, each scaled by what the same counter reads for a 1 GiB copy), and where the figure comes
    from.  It is not measured in this run, so it only counts while the kernel is what it was when the counters were
    read: the file records the hash of the kernel's sources, and with any other hash (or none) the bytes are None."""
    name = f"{kernel}_{workload.replace('-', '_')}_traffic.json"
    source = {"file": f"profiles/{name}", "measured_in_this_run": False}
    try:
        with open(os.path.join(ROOT, "profiles", name)) as f:
            rec = json.load(f)
        nbytes = float(rec["hbm_bytes_per_launch"])
    except (OSError, KeyError, ValueError):
        return None, None
    source["git_head"] = rec.get("git_head")
    source["kernel_source_sha16"] = rec.get("kernel_source_sha16")
    source["current_kernel_source_sha16"] = kernel_source_sha16(kernel)
    source["stale"] = source["kernel_source_sha16"] != source["current_kernel_source_sha16"]
    return (None if source["stale"] else nbytes), source


def cpu_baseline(w, tens, sample_seqs):
    """Time the C restatement on the host for a subset of the batch's sequences (same pages, same queries)."""
    import torch
    from oracle import c_oracle

    tag = {"f32": 0, "bf16": 1, "fp8": 2, "int8": 3}
    threads = c_oracle.max_threads()
    idx = np.arange(min(sample_seqs, w.S))
    ctx = w.context_lens[idx]
    need = -(-ctx.astype(np.int64) // w.page_size)
    # compact host pool: the live pages of the sample, renumbered from 1
    ids = np.concatenate([w.block_tables[i, :n] for i, n in zip(idx, need)])
    bt = np.zeros((len(idx), w.max_pages_per_seq), dtype=np.int32)
    k = 1
    for r, n in enumerate(need):
        bt[r, :n] = np.arange(k, k + n)
        k += int(n)
    dev_ids = torch.from_numpy(np.concatenate([[0], ids]).astype(np.int64)).to(tens["kv_pages"].device)
    pool = tens["kv_pages"][dev_ids]
    raw_dtype = {1: torch.uint8, 2: torch.int16, 4: torch.float32}[pool.element_size()]
    pool_np = pool.view(raw_dtype).cpu().numpy()
    scales_np = None if tens["kv_scales"] is None else tens["kv_scales"][dev_ids].cpu().numpy()
    qsl = np.concatenate([[0], np.cumsum(w.q_lens[idx])]).astype(np.int32)
    q0 = w.query_start_loc
    rows = np.concatenate([np.arange(q0[i], q0[i + 1]) for i in idx])
    q = tens["query"][torch.from_numpy(rows).to(tens["query"].device)]
    q_np = q.view(torch.int16 if q.element_size() == 2 else torch.float32).cpu().numpy()

    def run():
        return c_oracle.attention(q_np, tag[w.q_dtype], pool_np, tag[w.kv_dtype], scales_np, ctx, bt, qsl, [len(idx)],
                                  Hkv=w.Hkv, softmax_scale=w.softmax_scale, sliding_window=w.sliding_window,
                                  logits_soft_cap=w.logits_soft_cap, num_threads=threads)

    run()  # warm-up (page faults, thread pool)
    t0 = time.perf_counter()
    reps = 0
    while True:
        out = run()
        reps += 1
        if time.perf_counter() - t0 > 10.0:
            break
    dt = (time.perf_counter() - t0) / reps
    tokens = int(w.q_lens[idx].sum())
    return {
        "value": tokens / dt,
        "unit": "tokens/s (one attention-layer call)",
        "cores": threads,
        "kind": "port",
        "sample": f"first {len(idx)} of {w.S} sequences of the same batch ({int(ctx.sum())} cached tokens), "
                  f"C restatement with OpenMP, {reps} timed calls of {dt * 1e3:.1f} ms",
    }, out, rows


def bench_mla(args):
    """Multi-latent attention over latent pages (kv_lora_rank 512, rope 64, bf16, page size 64): a decode batch
    shaped like the default workload (256 sequences of 512..8192 tokens, one new token each) with 128 query heads
    (DeepSeek-V3 on one GPU) or 16 (its eighth, DeepSeek-V2-Lite), or a chunked prefill of 8 x 512 tokens after
    3 584.  One step = the fused call: page write + attention.  Same output line as the default workload; no CPU
    sample is timed for these."""
    import torch

    from easydel_amd import kernels

    dev = torch.device("cuda:0")
    rng = np.random.default_rng(args.seed)
    lkv, rope, row, pg = 512, 64, 640, 64
    if args.workload == "mla-prefill-h128":
        Hq, n = 128, 8
        q_lens = np.full(n, 512, np.int32)
        ctx = np.full(n, 4096, np.int32)
    else:
        Hq, n = (128 if args.workload.endswith("h128") else 16), 256
        q_lens = np.ones(n, np.int32)
        ctx = rng.integers(512, 8193, size=n).astype(np.int32)
        if args.mla_uniform_context > 0:
            ctx[:] = args.mla_uniform_context
    need = -(-ctx // pg)
    M = int(need.max())
    P = int(need.sum()) + 64
    perm = rng.permutation(np.arange(1, P)).astype(np.int32)
    bt = np.zeros((n, M), np.int32)
    k = 0
    for i, m in enumerate(need):
        bt[i, :m] = perm[k:k + m]
        k += m
    if args.mla_distinct_pages > 0 and args.workload != "mla-prefill-h128":
        bt = (bt % args.mla_distinct_pages).astype(np.int32)
    T = int(q_lens.sum())
    qsl = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    g = torch.Generator(device=dev).manual_seed(args.seed)
    rnd = lambda *shape: torch.randn(*shape, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)  # noqa: E731
    pages = torch.empty(P, pg, row, dtype=torch.bfloat16, device=dev)
    for lo in range(0, P, 4096):
        pages[lo:lo + 4096] = rnd(min(4096, P - lo), pg, row)
    qn, qp, kv, pe = rnd(T, Hq, lkv), rnd(T, Hq, rope), rnd(T, lkv), rnd(T, rope)
    i32 = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.int32)).to(dev)  # noqa: E731
    ctx_d, bt_d, qsl_d, dist_d = i32(ctx), i32(bt), i32(qsl), i32([0, 0, n])
    out = torch.empty_like(qn)
    scale = (128 + rope) ** -0.5

    def step(write=True):
        kernels.mla_ragged_paged_attention(qn, qp, kv if write else None, pe if write else None, pages, ctx_d, bt_d, qsl_d,
                                           dist_d, softmax_scale=scale, out=out)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    stream = torch.cuda.current_stream(dev)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for a, b in evs:  # the call without the page write: attention kernel + merge, bracketed on the launch stream
        a.record(stream)
        step(write=False)
        b.record(stream)
    torch.cuda.synchronize()
    att_ms = float(np.mean([a.elapsed_time(b) for a, b in evs]))
    # algorithmic bytes: every visible latent row once per sequence (it is key and value at once), queries, outputs,
    # block-table entries, lengths; flops: 2 (lkv + rope) for the scores + 2 lkv for the values, per (row, visible key)
    pos0 = ctx - q_lens
    pairs = int(sum(int(q) * int(p0) + int(q) * (int(q) + 1) // 2 for q, p0 in zip(q_lens, pos0)))
    nbytes = int(ctx.sum()) * (lkv + rope) * 2 + T * Hq * (2 * lkv + rope) * 2 + int(need.sum()) * 4 + (2 * n + 1) * 4
    flops = 2 * Hq * (2 * lkv + rope) * pairs
    hbm_frac = nbytes / (att_ms * 1e-3) / 1e9 / HBM_PEAK_GBS
    mfma_frac = flops / (att_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS
    bound = "hbm" if nbytes / (HBM_PEAK_GBS * 1e9) >= flops / (MFMA_BF16_PEAK_TFLOPS * 1e12) else "mfma"
    roofline = ({"bound": "hbm", "achieved": nbytes / (att_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": hbm_frac}
                if bound == "hbm" else
                {"bound": "mfma", "achieved": flops / (att_ms * 1e-3) / 1e12, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": mfma_frac})
    roofline.update({"traffic": None, "kernel": "mla_attn_kernel + mla_merge_kernel (the call without the page write)",
                     "kernel_ms": att_ms, "algorithmic_bytes_per_launch": nbytes, "algorithmic_flops_per_launch": flops,
                     "hbm_frac": hbm_frac, "mfma_frac": mfma_frac})
    print(json.dumps({
        "metric": "decode tokens/s + attn HBM TB/s (% of 8 TB/s), Llama-3-8B-shaped, 1 GPU",
        "value": T / (ms_per_step * 1e-3),
        "unit": "tokens/s (one attention-layer call: latent page write + multi-latent ragged paged attention)",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": args.workload, "sequences": n, "query_tokens": T, "q_heads": Hq, "kv_lora_rank": lkv,
                   "qk_rope_head_dim": rope, "page_row_elems": row, "page_size": pg, "pool_pages": P,
                   "context_tokens_total": int(ctx.sum()), "context_range": [int(ctx.min()), int(ctx.max())], "seed": args.seed,
                   "distinct_pages_in_block_tables": args.mla_distinct_pages or None},
        "roofline": roofline, "cpu_baseline": None,
    }))


def read_probe():
    """What the memory system gives a streaming reader: rpa_read_probe over 8 GiB, best of four timed launches."""
    import torch

    from easydel_amd import _lib

    lib = _lib.load()
    dev = torch.device("cuda:0")
    buf = torch.empty(8 << 30, dtype=torch.uint8, device=dev).fill_(1)
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream(dev)
    for wgs in (32, 64, 128, 192, 256):
        for kib in (2, 4, 8, 16, 32):
            best, read = None, 0
            for rep in range(5):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                read = lib.rpa_read_probe(stream.cuda_stream, buf.data_ptr(), buf.numel(), wgs, kib, sink.data_ptr())
                e1.record(stream)
                e1.synchronize()
                if read == 0:
                    raise RuntimeError(lib.rpa_last_error().decode())
                ms = e0.elapsed_time(e1)
                if rep > 0 and (best is None or ms < best):
                    best = ms
            print(json.dumps({"probe": "read", "workgroups": wgs, "kib_in_flight_per_workgroup": 8 * kib, "ms": round(best, 4),
                              "tb_per_s": round(read / best / 1e9, 3), "gb_per_s_per_workgroup": round(read / best / 1e6 / wgs, 1)}),
                  flush=True)


def read_probe_paged():
    """What the memory system gives the decode kernel's access pattern without its arithmetic: rpa_read_probe_paged over
    8 GiB (chunks visited in a scattered order, eight waves per chunk), best of four timed launches per setting."""
    import torch

    from easydel_amd import _lib

    lib = _lib.load()
    dev = torch.device("cuda:0")
    buf = torch.empty(8 << 30, dtype=torch.uint8, device=dev).fill_(1)
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream(dev)
    names = {0: "contiguous eighths, non-temporal loads", 1: "one head per wave, non-temporal loads", 2: "one head per wave, ordinary loads"}
    for chunk_kib, split in ((16, 0), (64, 0), (64, 1), (64, 2), (256, 0), (256, 1), (256, 2)):
        for wgs in (192, 256, 512):
            for kib in (2, 4, 8, 16, 32):
                if kib % (chunk_kib // 8):
                    continue
                best, read = None, 0
                for rep in range(5):
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record(stream)
                    read = lib.rpa_read_probe_paged(stream.cuda_stream, buf.data_ptr(), buf.numel(), wgs, kib, chunk_kib, split, sink.data_ptr())
                    e1.record(stream)
                    e1.synchronize()
                    if read == 0:
                        raise RuntimeError(lib.rpa_last_error().decode())
                    ms = e0.elapsed_time(e1)
                    if rep > 0 and (best is None or ms < best):
                        best = ms
                print(json.dumps({"probe": "read-paged", "chunk_kib": chunk_kib, "split": names[split], "workgroups": wgs,
                                  "kib_in_flight_per_workgroup": 8 * kib, "ms": round(best, 4), "tb_per_s": round(read / best / 1e9, 3),
                                  "gb_per_s_per_workgroup": round(read / best / 1e6 / wgs, 1)}), flush=True)


def mfma_probe():
    """What a stream of bf16 MFMAs sustains with its A operands in registers or read from LDS the way the prefill kernels
    read K and V tiles: rpa_mfma_probe, best of three timed launches per setting, with the clock the kernel ran at."""
    import torch

    from easydel_amd import _lib

    lib = _lib.load()
    dev = torch.device("cuda:0")
    clocks = torch.zeros(2, dtype=torch.int64, device=dev)
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream(dev)
    shapes = {0: "16x16x32", 1: "32x32x16"}
    sources = {0: "registers", 1: "LDS, ds_read_b128 (K pattern)", 2: "LDS, 2 x ds_read_b64_tr_b16 (V pattern)"}
    for source in (0, 1, 2):
        for shape in (0, 1):
            for reuse in (1, 2, 4):
                for waves in (1, 2):
                    iters = 8000 // reuse
                    best, flops, mhz = None, 0.0, 0.0
                    for rep in range(4):
                        clocks.zero_()
                        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                        e0.record(stream)
                        flops = lib.rpa_mfma_probe(stream.cuda_stream, shape, source, reuse, waves, iters, clocks.data_ptr(), sink.data_ptr())
                        e1.record(stream)
                        e1.synchronize()
                        if flops == 0.0:
                            raise RuntimeError(lib.rpa_last_error().decode())
                        ms = e0.elapsed_time(e1)
                        if rep > 0 and (best is None or ms < best):
                            best = ms
                            c = clocks.cpu().numpy()
                            mhz = 100.0 * float(c[0]) / float(c[1])
                    tf = flops / best / 1e9
                    print(json.dumps({"probe": "mfma", "shape": shapes[shape], "a_operands": sources[source], "mfmas_per_operand": reuse,
                                      "waves_per_simd": waves, "ms": round(best, 4), "tflop_per_s": round(tf, 1),
                                      "frac_of_2500": round(tf / MFMA_BF16_PEAK_TFLOPS, 4), "clock_mhz": round(mhz)}), flush=True)


def issue_probe():
    """Cycles per MFMA of a lone wave per SIMD that issues, beside every 32x32x16 bf16 MFMA, six independent v_fma_f32 (a
    full slot: MFMA 8 cycles of issue + 6 x 4) or none, and 0 / 1 / 2 / 4 instructions of one kind: rpa_issue_probe."""
    import torch

    from easydel_amd import _lib

    lib = _lib.load()
    dev = torch.device("cuda:0")
    clocks = torch.zeros(2, dtype=torch.int64, device=dev)
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    src = torch.ones(1 << 18, dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream(dev)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    kinds = ["v_fma_f32", "v_exp_f32", "v_rcp_f32", "v_cvt_pk_bf16_f32", "v_max3_f32 (dependent chain)", "s_add_u32 (dependent chain)", "s_nop 0",
             "ds_read_b128", "ds_read_b64_tr_b16", "global_load_lds_dwordx4 (m0 written each time)"]
    for kind, name in enumerate(kinds):
        rec = {"probe": "issue", "instruction": name}
        for fill in (6, 0):
            cyc = {}
            for extra in (0, 1, 2, 4):
                best = None
                for rep in range(3):
                    clocks.zero_()
                    n = lib.rpa_issue_probe(stream.cuda_stream, kind, extra, fill, 1000, clocks.data_ptr(), sink.data_ptr(), src.data_ptr())
                    if n == 0:
                        raise RuntimeError(lib.rpa_last_error().decode())
                    torch.cuda.synchronize()
                    c = clocks.cpu().numpy()
                    v = float(c[0]) / (cus * n)
                    if rep > 0 and (best is None or v < best):
                        best = v
                        rec["clock_mhz"] = round(100.0 * float(c[0]) / float(c[1]))
                cyc[extra] = best
            key = "full_slot" if fill else "mfma_alone"
            rec[f"cycles_per_mfma_{key}"] = {str(k): round(v, 1) for k, v in cyc.items()}
            if fill:
                rec["cycles_each_in_a_full_slot"] = round((cyc[4] - cyc[0]) / 4.0, 1)
        print(json.dumps(rec), flush=True)


_KEEP = []


def measure(args, workload, with_cpu):
    """One workload: the whole step timed on the host clock around synchronised launches, its kernels timed alone with
    events on the launch stream, and (with_cpu) the C restatement timed on the host cores.  Returns the result record."""
    import torch

    import bench_workloads as workloads
    from easydel_amd import _lib, kernels

    dev = torch.device("cuda:0")
    w = build_workload(workload, args.seed, args.sequential_pages, (args.chunk_seqs, args.chunk_len))
    if args.chunk_window > 0 and workload in ("fp8-prefill", "int8-prefill", "int8-prefill-d256", "int8-prefill-d256-cap"):
        import dataclasses

        w = dataclasses.replace(w, sliding_window=args.chunk_window)
    tens = workloads.device_tensors(w, dev, seed=args.seed)
    quant = w.kv_dtype in ("fp8", "int8")
    out = torch.empty_like(tens["query"])

    unified = args.layout == "unified"
    if unified:
        from easydel_amd.caching import compute_slot_mapping_v2

        key_cache = tens["kv_pages"][:, :, 0::2].contiguous()
        value_cache = tens["kv_pages"][:, :, 1::2].contiguous()
        # The interleaved pool stays allocated: returning a block of this size to the driver (empty_cache) leaves
        # the process in a state in which every kernel here runs about 3 % slower (measured: 742 -> 765 us for the
        # interleaved decode kernel, 775 -> 805 us for this layout's), and a serving process does not free its pools.
        slots_np, n_slices = compute_slot_mapping_v2(num_requests=w.S, scheduled=w.q_lens, num_computed_tokens=w.context_lens - w.q_lens,
                                                     page_table=w.block_tables, page_size=w.page_size)
        slots = torch.from_numpy(slots_np).to(dev)
        n_slices_dev = torch.tensor([n_slices], dtype=torch.int32, device=dev)
        k_flat, v_flat = key_cache.view(-1, w.Hkv, w.D), value_cache.view(-1, w.Hkv, w.D)
        args.no_cpu_baseline = True  # the host sample is cut from the interleaved pool

    def step():
        if unified:
            if not quant:
                kernels.page_scatter_slices(tens["key"], slots, n_slices_dev, k_flat, page_size=w.page_size)
                kernels.page_scatter_slices(tens["value"], slots, n_slices_dev, v_flat, page_size=w.page_size)
            kernels.unified_attention(tens["query"], key_cache, value_cache, tens["context_lens"], tens["block_tables"],
                                      tens["query_start_loc"], tens["num_seqs"], softmax_scale=w.softmax_scale,
                                      sliding_window=w.sliding_window, logits_soft_cap=w.logits_soft_cap,
                                      kv_scales=tens["kv_scales"], out=out)
        elif quant:  # scaled 8-bit pages: quantising write of the new rows, then the attention
            kernels.ragged_paged_attention_v3_quantised(tens["query"], tens["key"], tens["value"], tens["kv_pages"],
                                                        tens["kv_scales"], tens["context_lens"], tens["block_tables"],
                                                        tens["query_start_loc"], tens["distribution"],
                                                        softmax_scale=w.softmax_scale, sliding_window=w.sliding_window,
                                                        logits_soft_cap=w.logits_soft_cap, num_kv_heads=w.Hkv, out=out)
        else:
            kernels.ragged_paged_attention_v3(tens["query"], tens["key"], tens["value"], tens["kv_pages"],
                                              tens["context_lens"], tens["block_tables"], tens["query_start_loc"],
                                              tens["distribution"], softmax_scale=w.softmax_scale,
                                              sliding_window=w.sliding_window, logits_soft_cap=w.logits_soft_cap, out=out)

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):  # rpa::calibration_copy_kernel: reads 1 GiB, writes 1 GiB
            _lib.check(_lib.load().rpa_calibration_copy(torch.cuda.current_stream(dev).cuda_stream, dst.data_ptr(),
                                                        src.data_ptr(), src.numel()))
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # the same step recorded once in a HIP graph and replayed: what a serving loop that captures its decode step pays
    # (the library's launches are plain kernels on the caller's stream; its workspace was sized by the calls above)
    graph_ms = None
    if args.hip_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step()
        for _ in range(args.warmup):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        del graph

    # kernels in isolation: one call that only runs the plan kernel, then calls that launch only the decode
    # kernel (it reuses the plan left in the workspace) or only the prefill kernel, bracketed by events on the
    # launch stream
    stream = torch.cuda.current_stream(dev)
    if unified:
        att = lambda: kernels.unified_attention(  # noqa: E731
            tens["query"], key_cache, value_cache, tens["context_lens"], tens["block_tables"], tens["query_start_loc"],
            tens["num_seqs"], softmax_scale=w.softmax_scale, sliding_window=w.sliding_window,
            logits_soft_cap=w.logits_soft_cap, kv_scales=tens["kv_scales"], out=out)
    else:
        att = lambda: kernels.ragged_paged_attention(  # noqa: E731
            tens["query"], tens["kv_pages"], tens["context_lens"], tens["block_tables"], tens["query_start_loc"],
            tens["num_seqs"], softmax_scale=w.softmax_scale, sliding_window=w.sliding_window,
            logits_soft_cap=w.logits_soft_cap, kv_scales=tens["kv_scales"], num_kv_heads=w.Hkv, out=out)

    def time_stage(mask, reps):
        _lib.set_tunable("stages", mask)
        for _ in range(3):
            att()
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
        for a, b in evs:
            a.record(stream)
            att()
            b.record(stream)
        torch.cuda.synchronize()
        return float(np.mean([a.elapsed_time(b) for a, b in evs]))

    prev = _lib.set_tunable("stages", 1)
    att()
    small = w.small_row_mask()
    kern = {}
    if small.any():
        ms = time_stage(2, args.steps)
        nbytes = w.attention_bytes(small)
        kern["attn_decode_kernel"] = {
            "bound": "hbm", "achieved": nbytes / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None, "traffic_source": None,
            "algorithmic_bytes_per_launch": nbytes, "kernel_ms": ms}
        if not unified:
            kern["attn_decode_kernel"]["traffic"], kern["attn_decode_kernel"]["traffic_source"] = measured_traffic(workload)
    if (~small & (w.q_lens > 0)).any():
        ms = time_stage(4, args.steps)
        flops = w.attention_flops(~small)
        kern["attn_prefill_kernel"] = {
            "bound": "mfma", "achieved": flops / (ms * 1e-3) / 1e12, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": flops / (ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, "traffic": None, "traffic_source": None,
            "algorithmic_flops_per_launch": flops, "algorithmic_bytes_per_launch": w.attention_bytes(~small),
            "kernel_ms": ms}
        if not unified:
            kern["attn_prefill_kernel"]["traffic"], kern["attn_prefill_kernel"]["traffic_source"] = \
                measured_traffic(workload, "attn_prefill_kernel")
    _lib.set_tunable("stages", prev)
    dominant = max(kern, key=lambda k: kern[k]["kernel_ms"])
    roofline = dict(kern[dominant], kernel=dominant)
    att_bytes = w.attention_bytes()

    result = {
        "metric": "decode tokens/s + attn HBM TB/s (% of 8 TB/s), Llama-3-8B-shaped, 1 GPU",
        "value": w.T / (ms_per_step * 1e-3),
        "unit": "tokens/s (one attention-layer call: page scatter + ragged paged attention)",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "ms_per_step_hip_graph": graph_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": {"bf16": "bf16", "fp8": "bf16 x fp8-e4m3 KV", "int8": "bf16 x int8 KV"}[w.kv_dtype],
        "data": "synthetic",
        "config": {
            "workload": w.name,
            "kv_layout": args.layout,
            "sequences": w.S,
            "query_tokens": w.T,
            "q_heads": w.Hq,
            "kv_heads": w.Hkv,
            "head_dim": w.D,
            "page_size": w.page_size,
            "pool_pages": w.num_pages,
            "context_tokens_total": int(w.context_lens.sum()),
            "context_range": [int(w.context_lens.min()), int(w.context_lens.max())],
            "sliding_window": w.sliding_window,
            "logits_soft_cap": w.logits_soft_cap,
            "seed": args.seed,
        },
        "attention_only_model_tokens_per_s_32_layers": w.T / (ms_per_step * 1e-3) / 32.0,
        "step_hbm_tb_s": (att_bytes + w.scatter_bytes()) / (ms_per_step * 1e-3) / 1e12,
        "roofline": roofline,
        "kernels": kern,
    }
    if "attn_decode_kernel" in kern:
        result["attn_hbm_tb_s"] = kern["attn_decode_kernel"]["achieved"] / 1e3
        result["attn_hbm_pct_of_8tb_s"] = 100.0 * kern["attn_decode_kernel"]["frac"]

    if with_cpu and not args.no_cpu_baseline:
        # the whole batch fits the host here; it is re-run for about 10 s
        sample = args.cpu_sample_seqs or w.S
        base, cpu_out, rows = cpu_baseline(w, tens, sample)
        step()
        torch.cuda.synchronize()
        gpu_rows = out[torch.from_numpy(rows).to(dev)].float().cpu().numpy()
        base["max_abs_diff_vs_gpu_on_sample"] = float(np.abs(gpu_rows - cpu_out).max())
        result["cpu_baseline"] = base
    else:
        result["cpu_baseline"] = None

    _KEEP.append((tens, out))  # pools stay allocated: handing blocks of this size back to the driver slows later kernels by a few percent
    return result



def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    import bench_workloads as workloads
    from easydel_amd import _lib, kernels

    _lib.load()
    if args.read_probe:
        return read_probe()
    if args.read_probe_paged:
        return read_probe_paged()
    if args.mfma_probe:
        return mfma_probe()
    if args.issue_probe:
        return issue_probe()
    if args.workload.startswith("mla-"):
        if args.mla_chunks:
            _lib.set_tunable("mla_chunks", args.mla_chunks)
        if args.mla_min_chunk:
            _lib.set_tunable("mla_min_chunk", args.mla_min_chunk)
        return bench_mla(args)
    if args.decode_wgs:
        _lib.set_tunable("decode_wgs", args.decode_wgs)
    if args.decode_sync >= 0:
        _lib.set_tunable("decode_sync", args.decode_sync)
    if args.decode_dma >= 0:
        _lib.set_tunable("decode_dma", args.decode_dma)
    if args.prefill_chunks:
        _lib.set_tunable("prefill_chunks", args.prefill_chunks)
    if args.max_splits:
        _lib.set_tunable("max_splits", args.max_splits)
    if args.prefill_x32 >= 0:
        _lib.set_tunable("prefill_x32", args.prefill_x32)
    if args.prefill_wide >= 0:
        _lib.set_tunable("prefill_wide", args.prefill_wide)

    result = measure(args, args.workload, True)
    if args.workload == "c2" and args.layout == "interleaved" and not args.no_extra_configs:
        # the other benchmark configurations, each with its step time and its dominant kernel against its roofline
        # (no host leg for them); the headline fields above stay those of the decode configuration
        def record(name):
            r = measure(args, name, False)
            roof = r["roofline"]
            rec = {"workload": r["config"]["workload"], "ms_per_step": r["ms_per_step"], "tokens_per_s": r["value"], "dtype": r["dtype"],
                   "kernel": roof["kernel"], "kernel_ms": roof["kernel_ms"],
                   "roofline": {k: roof[k] for k in ("bound", "achieved", "peak", "unit", "frac", "traffic")},
                   "traffic_source": roof.get("traffic_source"), "kernels_ms": {k: v["kernel_ms"] for k, v in r["kernels"].items()}}
            for key in ("algorithmic_bytes_per_launch", "algorithmic_flops_per_launch"):
                if key in roof:
                    rec[key.replace("_per_launch", "")] = roof[key]
            return rec

        result["configs"] = {name: record(name) for name in ("c3", "c4-fp8", "c4-int8", "c5-global", "c5-window")}
        # two shapes that are none of the benchmark's, in the same form: the prefill kernel on a batch that fills the chip,
        # and prompt chunks over scaled fp8 pages (the prefill stage there: decision, page copy, the kernel on the copies)
        result["tuning_shapes"] = {name: record(name) for name in ("llama-prefill", "fp8-prefill")}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
