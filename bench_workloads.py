"""Seeded synthetic workloads of the five benchmark shapes (metadata in numpy, page pools on the GPU).

Metadata follows the reference's serving conventions: page 0 is the null page and never handed to a
sequence (easydel/inference/esurge/core/page_pool.py:87-88), block-table rows are padded with 0
(page_table.py:48-49), ``query_start_loc`` is extended flat past the live rows
(runners/executors/batch_preparer.py:618-621), decode rows come first and
``distribution = [n_decode, n_decode + n_prefill, n_total]`` (batch_preparer.py:698-709).
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np


@dataclass
class Workload:
    name: str
    Hq: int
    Hkv: int
    D: int
    page_size: int
    num_pages: int
    max_pages_per_seq: int
    context_lens: np.ndarray  # int32 [S], new tokens included
    q_lens: np.ndarray  # int32 [S]
    block_tables: np.ndarray  # int32 [S, M]
    q_dtype: str = "bf16"
    kv_dtype: str = "bf16"  # "f32" | "bf16" | "fp8" | "int8"
    softmax_scale: float | None = None
    sliding_window: int | None = None
    logits_soft_cap: float | None = None
    extra: dict = field(default_factory=dict)

    @property
    def S(self) -> int:
        return len(self.context_lens)

    @property
    def T(self) -> int:
        return int(self.q_lens.sum())

    @property
    def query_start_loc(self) -> np.ndarray:
        return np.concatenate([[0], np.cumsum(self.q_lens)]).astype(np.int32)

    @property
    def num_seqs(self) -> np.ndarray:
        return np.array([int((self.q_lens > 0).sum())], dtype=np.int32)

    @property
    def distribution(self) -> np.ndarray:
        has = self.q_lens > 0
        dec = (self.q_lens == 1) & (self.context_lens > 1) & has
        return np.array([dec.sum(), dec.sum() + (has & ~dec).sum(), has.sum()], dtype=np.int32)

    @property
    def kv_elem_bytes(self) -> int:
        return {"f32": 4, "bf16": 2, "fp8": 1, "int8": 1}[self.kv_dtype]

    @property
    def q_elem_bytes(self) -> int:
        return {"f32": 4, "bf16": 2}[self.q_dtype]

    def visible_keys(self) -> np.ndarray:
        """Keys each sequence must read: ctx, or min(ctx, W + q_len - 1) under a window."""
        ctx = self.context_lens.astype(np.int64)
        if self.sliding_window:
            return np.minimum(ctx, self.sliding_window + self.q_lens.astype(np.int64) - 1)
        return ctx

    def decode_row_limit(self) -> int:
        """Most (token, group-head) rows per KV head of a sequence the split-K decode kernel serves in a call on this
        workload: 32 for bf16 pages up to head size 128 when the batch has more query tokens than sequence rows
        (only then can a row hold several tokens), else 16 (mirrors ``decode_row_limit`` of the library)."""
        return 32 if (self.kv_dtype == "bf16" and self.D <= 128 and int(self.q_lens.sum()) > len(self.q_lens)) else 16

    def small_row_mask(self) -> np.ndarray:
        """Sequences the split-K decode kernel serves."""
        return (self.q_lens > 0) & (self.q_lens * (self.Hq // self.Hkv) <= self.decode_row_limit())

    def attention_bytes(self, select: np.ndarray | None = None) -> int:
        """Algorithmic HBM bytes of one attention call: every visible K/V element once per sequence,
        q and out once, the block-table entries and lengths that are consulted, per-page scales if any.
        ``select`` restricts the count to a subset of sequences (boolean mask)."""
        live = self.q_lens > 0
        if select is not None:
            live = live & select
        vis = self.visible_keys()[live]
        kv = int(vis.sum()) * self.Hkv * self.D * 2 * self.kv_elem_bytes
        qo = int(self.q_lens[live].sum()) * self.Hq * self.D * 2 * self.q_elem_bytes
        pages = int(np.ceil(vis / self.page_size).sum())
        meta = pages * 4 + (2 * self.S + 1) * 4
        scales = pages * 2 * self.Hkv * 4 if self.kv_dtype in ("fp8", "int8") else 0
        return kv + qo + meta + scales

    def scatter_bytes(self) -> int:
        """Read + write of the new K/V rows."""
        return 2 * self.T * 2 * self.Hkv * self.D * self.kv_elem_bytes

    def attention_flops(self, select: np.ndarray | None = None) -> int:
        """4 * Hq * D flops per visible (query row, key) pair."""
        pairs = 0
        for k, (ctx, ql) in enumerate(zip(self.context_lens.astype(np.int64), self.q_lens.astype(np.int64))):
            if ql <= 0 or (select is not None and not select[k]):
                continue
            pos = ctx - ql + np.arange(ql)
            n = pos + 1
            if self.sliding_window:
                n = np.minimum(n, self.sliding_window)
            pairs += int(n.sum())
        return 4 * self.Hq * self.D * pairs


def _tables(rng, context_lens, page_size, num_pages, max_pages, shuffle=True):
    """Consecutive slices of one seeded permutation of pages 1..P-1 (no page shared)."""
    need = -(-context_lens.astype(np.int64) // page_size)
    if need.sum() > num_pages - 1:
        raise ValueError(f"pool of {num_pages} pages cannot hold {int(need.sum())} live pages")
    perm = rng.permutation(np.arange(1, num_pages, dtype=np.int32)) if shuffle else np.arange(1, num_pages, dtype=np.int32)
    bt = np.zeros((len(context_lens), max_pages), dtype=np.int32)
    k = 0
    for i, n in enumerate(need):
        bt[i, :n] = perm[k:k + n]
        k += int(n)
    return bt


def config1_tiny_mixed(seed: int = 0) -> Workload:
    rng = np.random.default_rng(seed)
    ctx = np.array([17, 64, 130, 255], dtype=np.int32)
    return Workload("C1 tiny fp32 mixed batch", Hq=8, Hkv=2, D=64, page_size=16, num_pages=128, max_pages_per_seq=16,
                    context_lens=ctx, q_lens=np.array([1, 1, 8, 33], dtype=np.int32),
                    block_tables=_tables(rng, ctx, 16, 128, 16), q_dtype="f32", kv_dtype="f32", softmax_scale=1.0 / 8.0)


def config2_llama_decode(seed: int = 0, n_seqs: int = 256, num_pages: int = 40_000, shuffle_pages: bool = True) -> Workload:
    rng = np.random.default_rng(seed)
    ctx = rng.integers(512, 8193, size=n_seqs).astype(np.int32)
    return Workload("C2 Llama-3-8B-shaped pure decode", Hq=32, Hkv=8, D=128, page_size=64, num_pages=num_pages,
                    max_pages_per_seq=128, context_lens=ctx, q_lens=np.ones(n_seqs, dtype=np.int32),
                    block_tables=_tables(rng, ctx, 64, num_pages, 128, shuffle_pages), softmax_scale=128.0 ** -0.5)


def decode_shape(seed: int = 0, *, Hq: int = 32, Hkv: int = 8, n_seqs: int = 256, num_pages: int | None = None) -> Workload:
    """Not one of the five benchmark shapes: the pure-decode batch of C2 (contexts of 512..8192 tokens, head size 128,
    64-token pages) at other head counts -- 28 / 4 and 8 / 1, the shards of a Qwen-shaped and a Llama-70B-shaped model under
    tensor parallelism over the KV heads -- or at other batch sizes (16 and 32 sequences, where the call is launch-bound)."""
    rng = np.random.default_rng(seed)
    ctx = rng.integers(512, 8193, size=n_seqs).astype(np.int32)
    pages = num_pages if num_pages is not None else int(np.ceil(ctx / 64).sum()) + 64
    return Workload(f"pure decode, {Hq}/{Hkv} heads, {n_seqs} sequences (tuning shape)", Hq=Hq, Hkv=Hkv, D=128, page_size=64,
                    num_pages=pages, max_pages_per_seq=128, context_lens=ctx, q_lens=np.ones(n_seqs, dtype=np.int32),
                    block_tables=_tables(rng, ctx, 64, pages, 128), softmax_scale=128.0 ** -0.5)


def config3_mixed_chunked(seed: int = 0, num_pages: int = 48_000) -> Workload:
    rng = np.random.default_rng(seed)
    dec = rng.integers(1024, 16385, size=64)
    prior = rng.integers(0, 30721, size=4)
    ctx = np.concatenate([dec, prior + 512]).astype(np.int32)
    q_lens = np.concatenate([np.ones(64), np.full(4, 512)]).astype(np.int32)
    return Workload("C3 mixed chunked-prefill + decode, Llama-3-8B-shaped", Hq=32, Hkv=8, D=128, page_size=64,
                    num_pages=num_pages, max_pages_per_seq=512, context_lens=ctx, q_lens=q_lens,
                    block_tables=_tables(rng, ctx, 64, num_pages, 512), softmax_scale=128.0 ** -0.5)


def config4_quantised_decode(seed: int = 0, kv_dtype: str = "fp8", n_seqs: int = 512, num_pages: int = 140_000) -> Workload:
    rng = np.random.default_rng(seed)
    ctx = rng.integers(4096, 16385, size=n_seqs).astype(np.int32)
    return Workload(f"C4 Qwen2.5-32B-shaped {kv_dtype}-KV decode", Hq=40, Hkv=8, D=128, page_size=64, num_pages=num_pages,
                    max_pages_per_seq=256, context_lens=ctx, q_lens=np.ones(n_seqs, dtype=np.int32),
                    block_tables=_tables(rng, ctx, 64, num_pages, 256), kv_dtype=kv_dtype, softmax_scale=128.0 ** -0.5)


def config5_gemma_long_prefill(seed: int = 0, windowed: bool = False, num_pages: int = 2048) -> Workload:
    rng = np.random.default_rng(seed)
    ctx = np.array([61_440 + 2048, 126_976 + 2048], dtype=np.int32)
    return Workload("C5 Gemma-2-9B-shaped long-context chunked prefill" + (" (window 4096)" if windowed else " (global)"),
                    Hq=16, Hkv=8, D=256, page_size=128, num_pages=num_pages, max_pages_per_seq=1008, context_lens=ctx,
                    q_lens=np.array([2048, 2048], dtype=np.int32), block_tables=_tables(rng, ctx, 128, num_pages, 1008),
                    softmax_scale=1.0 / 16.0, sliding_window=4096 if windowed else None, logits_soft_cap=50.0)


def llama_long_prefill(seed: int = 0, n_seqs: int = 8, q_len: int = 2048, num_pages: int = 6000) -> Workload:
    """Not one of the five benchmark shapes: a prefill batch large enough to fill the chip at head size 128 (the
    mixed shape C3 holds only 4 x 512 prefill tokens), used to tune and profile the prefill kernel."""
    rng = np.random.default_rng(seed)
    prior = rng.integers(8192, 32769, size=n_seqs)
    ctx = (prior + q_len).astype(np.int32)
    return Workload("Llama-3-8B-shaped long-context chunked prefill (tuning shape)", Hq=32, Hkv=8, D=128, page_size=64,
                    num_pages=num_pages, max_pages_per_seq=576, context_lens=ctx, q_lens=np.full(n_seqs, q_len, dtype=np.int32),
                    block_tables=_tables(rng, ctx, 64, num_pages, 576), softmax_scale=128.0 ** -0.5)


def gemma_decode(seed: int = 0, n_seqs: int = 256, num_pages: int = 12_000) -> Workload:
    """Not one of the five benchmark shapes: pure decode at the heads of the long-context prefill configuration (16
    query heads over 8 KV heads, head size 256, 128-token pages, soft cap 50), ``n_seqs`` sequences of 512..8192 tokens.
    The decode shape on which the library picks its LDS-direct decode kernel."""
    rng = np.random.default_rng(seed)
    ctx = rng.integers(512, 8193, size=n_seqs).astype(np.int32)
    return Workload("Gemma-2-9B-shaped pure decode (tuning shape)", Hq=16, Hkv=8, D=256, page_size=128, num_pages=num_pages,
                    max_pages_per_seq=64, context_lens=ctx, q_lens=np.ones(n_seqs, dtype=np.int32),
                    block_tables=_tables(rng, ctx, 128, num_pages, 64), softmax_scale=1.0 / 16.0, logits_soft_cap=50.0)


def quantised_long_prefill(seed: int = 0, kv_dtype: str = "fp8", n_seqs: int = 4, q_len: int = 2048, num_pages: int = 2000,
                           head_dim: int = 128, soft_cap: float | None = None) -> Workload:
    """Not one of the five benchmark shapes: chunked prefill over scaled 8-bit pages at the heads of the quantised decode
    configuration (40 query heads, 8 KV heads, head size 128, 64-token pages): ``n_seqs`` chunks of ``q_len`` tokens
    appended to 8192..16384 tokens of context.  Used to measure the 8-bit prefill kernel.  ``head_dim`` 256: the same at
    16 query heads over 8 KV heads of 256 (a Gemma-shaped global-attention layer), with ``soft_cap`` or without."""
    rng = np.random.default_rng(seed)
    prior = rng.integers(8192 - q_len, 16385 - q_len, size=n_seqs)
    ctx = (prior + q_len).astype(np.int32)
    if head_dim == 256:
        return Workload(f"Gemma-shaped (head size 256, {'soft cap %g' % soft_cap if soft_cap else 'no soft cap'}) {kv_dtype}-KV chunked prefill (tuning shape)",
                        Hq=16, Hkv=8, D=256, page_size=64, num_pages=num_pages, max_pages_per_seq=256, context_lens=ctx,
                        q_lens=np.full(n_seqs, q_len, dtype=np.int32), block_tables=_tables(rng, ctx, 64, num_pages, 256), kv_dtype=kv_dtype,
                        softmax_scale=256.0 ** -0.5, logits_soft_cap=soft_cap)
    return Workload(f"Qwen2.5-32B-shaped {kv_dtype}-KV chunked prefill (tuning shape)", Hq=40, Hkv=8, D=128, page_size=64,
                    num_pages=num_pages, max_pages_per_seq=256, context_lens=ctx, q_lens=np.full(n_seqs, q_len, dtype=np.int32),
                    block_tables=_tables(rng, ctx, 64, num_pages, 256), kv_dtype=kv_dtype, softmax_scale=128.0 ** -0.5)


# ---- device side ---------------------------------------------------------------------------------


def _torch_dtype(name: str):
    import torch

    return {"f32": torch.float32, "bf16": torch.bfloat16, "fp8": torch.float8_e4m3fn, "int8": torch.int8}[name]


def device_tensors(w: Workload, device="cuda:0", seed: int = 0) -> dict:
    """Random-normal queries / new K,V / page pool on the GPU, plus the metadata arrays.

    fp8 pools hold e4m3 codes of N(0,1) with per-(page, combined head) scales ~ U[0.5, 2.0]; int8 pools hold
    symmetric codes of N(0,1)*s with scale = amax/127 per (page, combined head).
    """
    import torch

    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    C = 2 * w.Hkv
    kvt = _torch_dtype(w.kv_dtype)
    pool = torch.empty((w.num_pages, w.page_size, C, w.D), dtype=kvt, device=device)
    scales = None
    if w.kv_dtype in ("fp8", "int8"):
        scales = torch.empty((w.num_pages, C), dtype=torch.float32, device=device)
    step = max(1, (256 << 20) // (w.page_size * C * w.D * 4))  # ~256 MiB of fp32 noise at a time
    for p0 in range(0, w.num_pages, step):
        p1 = min(w.num_pages, p0 + step)
        noise = torch.randn((p1 - p0, w.page_size, C, w.D), dtype=torch.float32, device=device, generator=gen)
        if w.kv_dtype == "fp8":
            scales[p0:p1] = torch.rand((p1 - p0, C), device=device, generator=gen) * 1.5 + 0.5
            pool[p0:p1] = noise.to(kvt)
        elif w.kv_dtype == "int8":
            s = torch.rand((p1 - p0, 1, C, 1), device=device, generator=gen) * 1.5 + 0.5
            true = noise * s
            sc = true.abs().amax(dim=(1, 3)) / 127.0
            scales[p0:p1] = sc
            pool[p0:p1] = torch.clamp(torch.round(true / sc[:, None, :, None]), -127, 127).to(kvt)
        else:
            pool[p0:p1] = noise.to(kvt)
        del noise
    qt = _torch_dtype(w.q_dtype)
    T = w.T
    tens = {
        "query": torch.randn((T, w.Hq, w.D), dtype=torch.float32, device=device, generator=gen).to(qt),
        "key": torch.randn((T, w.Hkv, w.D), dtype=torch.float32, device=device, generator=gen),
        "value": torch.randn((T, w.Hkv, w.D), dtype=torch.float32, device=device, generator=gen),
        "kv_pages": pool,
        "kv_scales": scales,
        "context_lens": torch.from_numpy(w.context_lens).to(device),
        "block_tables": torch.from_numpy(w.block_tables).to(device),
        "query_start_loc": torch.from_numpy(w.query_start_loc).to(device),
        "num_seqs": torch.from_numpy(w.num_seqs).to(device),
        "distribution": torch.from_numpy(w.distribution).to(device),
    }
    if w.kv_dtype in ("f32", "bf16"):
        tens["key"] = tens["key"].to(kvt)
        tens["value"] = tens["value"].to(kvt)
    return tens
