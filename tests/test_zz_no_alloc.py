"""The entry point that allocates nothing (rpa_ragged_paged_attention_v3_static: scratch in a device array inside the
library) against the entry point it is a variant of, through the C ABI: two calls in a row, the second on a smaller
batch, each compared with rpa_ragged_paged_attention_v3 on the same inputs."""

import numpy as np
import pytest
import torch

import rpa_testlib as tl
from easydel_amd import _lib, kernels
from rpa_testlib import BF16, orc

pytestmark = pytest.mark.gpu
STATIC_BYTES = 64 << 20


def _case(seed, ctx, q_lens, gpu, **shape):
    b = tl.make_batch(seed, ctx, q_lens, pad_rows=1, pad_tokens=2, **shape)
    rng = np.random.default_rng(seed + 1)
    key_raw = orc.f32_to_bf16_bits(rng.standard_normal((b.T, b.Hkv, b.D), dtype=np.float32))
    val_raw = orc.f32_to_bf16_bits(rng.standard_normal((b.T, b.Hkv, b.D), dtype=np.float32))
    d = tl.device_batch(b, gpu)
    d["key"], d["value"] = tl.to_torch(key_raw, BF16, gpu), tl.to_torch(val_raw, BF16, gpu)
    d["dist"] = torch.tensor([0, 0, b.n], dtype=torch.int32, device=gpu)
    want_pages = orc.page_scatter_ragged_ref(key_raw, val_raw, b.kv_raw, b.context_lens, b.block_tables, b.query_start_loc, b.num_seqs)
    return b, d, want_pages


def _call_existing(b, d, ws):
    """rpa_ragged_paged_attention_v3 with a caller-owned workspace of ws.numel() bytes, on a copy of the pool."""
    lib = _lib.load()
    pages, out = d["kv_pages"].clone(), torch.full_like(d["query"], float("nan"))
    T, Hq, D = d["query"].shape
    _lib.check(lib.rpa_ragged_paged_attention_v3(
        torch.cuda.current_stream().cuda_stream, d["query"].data_ptr(), d["key"].data_ptr(), d["value"].data_ptr(), pages.data_ptr(),
        d["context_lens"].data_ptr(), d["block_tables"].data_ptr(), d["query_start_loc"].data_ptr(), d["dist"].data_ptr(),
        out.data_ptr(), ws.data_ptr(), ws.numel(), T, b.S, b.M, b.P, b.page_size, Hq, b.Hkv, D, D, b.C, 1, 1, D ** -0.5, 0, 0.0, None))
    torch.cuda.synchronize()
    return out, pages


def test_static_workspace_entry_point_matches_the_one_it_is_a_variant_of(gpu):
    shape = dict(Hq=32, Hkv=8, D=128, page_size=64)
    # first call: decode rows cut into several partial slots, multi-token rows, a prefill chunk split over keys;
    # second call: a smaller batch (fewer sequences, tokens and pages), whose partial slots overlay the first call's
    cases = [_case(900, [9000, 700, 65, 1500, 300, 12000, 4100], [1, 1, 1, 2, 150, 1, 700], gpu, **shape),
             _case(910, [700, 65, 2100], [1, 1, 40], gpu, **shape)]
    same_size_ws = torch.empty(STATIC_BYTES + 256, dtype=torch.uint8, device=gpu)
    ws_ptr = (same_size_ws.data_ptr() + 255) & ~255  # the library aligns the base itself; keep the byte count equal
    aligned = same_size_ws[ws_ptr - same_size_ws.data_ptr():][:STATIC_BYTES]
    for n, (b, d, want_pages) in enumerate(cases):
        T, Hq, D = d["query"].shape
        full = kernels.workspace_bytes(T, b.S, b.M, b.page_size, Hq, b.Hkv, D, torch.bfloat16, torch.bfloat16)
        want_full, pages_full = _call_existing(b, d, torch.empty(full, dtype=torch.uint8, device=gpu))
        want_same, pages_same = _call_existing(b, d, aligned)
        pages, out = d["kv_pages"].clone(), torch.full_like(d["query"], float("nan"))
        before = torch.cuda.memory_allocated(gpu)
        kernels.ragged_paged_attention_v3_static(d["query"], d["key"], d["value"], pages, d["context_lens"], d["block_tables"].reshape(-1),
                                                 d["query_start_loc"], d["dist"], out=out)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated(gpu) == before
        # the page write: bit-exact against the oracle and the existing entry point
        got_pages = pages.view(torch.int16).cpu().numpy().view(np.uint16)
        assert np.array_equal(got_pages, want_pages), f"call {n}: pages"
        assert torch.equal(pages, pages_full) and torch.equal(pages, pages_same)
        # the attention: the same bits as the existing entry point with a workspace of the same size (same layout),
        # within the bf16 tolerance of it with its own full-size workspace (more partial slots) and of the oracle
        rows = tl.valid_rows(b)
        assert torch.equal(out[rows], want_same[rows]), f"call {n}: output differs from the existing entry point"
        assert not out[rows.stop:].float().abs().sum().item(), "padded token rows must be zeros"
        got = tl.from_torch(out, BF16)
        tl.assert_close(got, tl.from_torch(want_full, BF16), b, f"call {n} vs full-size workspace")
        vals = orc.bf16_bits_to_f32(want_pages).astype(np.float64)
        tl.assert_close(got, tl.oracle_out(b, kv_val=vals), b, f"call {n} vs oracle")
        print(f"static workspace call {n}: T={T} full workspace {full >> 20} MiB, static {STATIC_BYTES >> 20} MiB: ok", flush=True)


def test_static_workspace_entry_point_rejects_shapes_beyond_its_array(gpu):
    lib = _lib.load()
    a = 0x7000_0000_0000  # never dereferenced: the size check comes first
    # 4096 decode-class tokens x 64 heads x 256 dims: two float32 partial slots alone are 512 MiB
    rc = lib.rpa_ragged_paged_attention_v3_static(None, a, a, a, a, a, a, a, a, a, 4096, 4096, 64, 1000, 64, 64, 8, 256, 256, 16, 1, 1,
                                                  0.0625, 0, 0.0, None)
    assert rc == _lib.RPA_ERR_WORKSPACE and b"built-in array holds 67108864" in lib.rpa_last_error()
    assert lib.rpa_ragged_paged_attention_v3_static(None, a, a, a, a, a, a, a, a, a, 0, 4, 4, 10, 64, 8, 2, 128, 128, 4, 1, 1,
                                                    0.1, 0, 0.0, None) == 0  # an empty batch is a no-op


def test_static_workspace_entry_point_replays_from_a_hip_graph(gpu):
    """What the entry point is for: a caller that may not allocate.  After one eager call (which looks up the array's
    address on this device) the call is captured into a HIP graph and replayed, with eager work and synchronisation
    between replays; every replay gives the eager result, and new metadata in the same buffers is picked up."""
    b, d, _ = _case(920, [3000, 700, 65, 1500, 300, 5000], [1, 1, 1, 2, 90, 1], gpu, Hq=32, Hkv=8, D=128, page_size=64)
    pages, out = d["kv_pages"].clone(), torch.empty_like(d["query"])

    def call():
        kernels.ragged_paged_attention_v3_static(d["query"], d["key"], d["value"], pages, d["context_lens"], d["block_tables"].reshape(-1),
                                                 d["query_start_loc"], d["dist"], out=out)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    eager = out.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        call()
    for rep in range(3):
        out.zero_()
        d["query"].mul_(1.0)  # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {rep} differs from the eager result"
    d["context_lens"][0] = 2900  # a shorter first sequence: its new token lands elsewhere and it sees fewer keys
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    replayed = out.clone()
    call()
    torch.cuda.synchronize()
    assert torch.equal(replayed, out), "a replay with new metadata differs from the eager call on the same buffers"
    assert not torch.equal(replayed[:1], eager[:1])
