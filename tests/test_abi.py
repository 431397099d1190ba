"""The C-ABI library loads and exports every symbol include/rpa_hip.h and include/rpa_hip_probe.h declare (no compute calls: no GPU here)."""

import ctypes
import os
import re

import pytest

from easydel_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    names = set()
    for header in ("rpa_hip.h", "rpa_hip_probe.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(rpa_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_header_symbols_are_exported_and_bound():
    names = _declared_symbols()
    assert {"rpa_ragged_paged_attention", "rpa_ragged_paged_attention_v3", "rpa_page_scatter_slices", "rpa_page_scatter_ragged",
            "rpa_attention_workspace_bytes", "rpa_version", "rpa_last_error", "rpa_set_tunable", "rpa_calibration_copy"} <= set(names)
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    for n in names:
        assert hasattr(lib, n), f"{n} declared in rpa_hip.h but not exported by librpa_hip.so"
        assert n in _lib.SIGNATURES or n in _lib.PROBE_SIGNATURES, f"{n} has no ctypes prototype in easydel_amd/_lib.py"
    assert sorted(list(_lib.SIGNATURES) + list(_lib.PROBE_SIGNATURES)) == names


def test_host_only_entry_points():
    lib = _lib.load()
    assert re.fullmatch(r"\d+\.\d+\.\d+", lib.rpa_version().decode())
    # argument validation happens before any device work
    rc = lib.rpa_ragged_paged_attention(None, None, None, None, None, None, None, None, None, None, 0,
                                        4, 1, 1, 1, 16, 8, 3, 64, 64, 6, 1, 1, 1.0, 0, 0.0, None)
    assert rc == _lib.RPA_ERR_INVALID_ARGUMENT and b"multiple of Hkv" in lib.rpa_last_error()
    rc = lib.rpa_ragged_paged_attention(None, None, None, None, None, None, None, None, None, None, 0,
                                        4, 1, 1, 1, 16, 8, 2, 64, 64, 4, 9, 1, 1.0, 0, 0.0, None)
    assert rc == _lib.RPA_ERR_UNSUPPORTED
    a = 0x7000_0000_0000
    rc = lib.rpa_ragged_paged_attention(None, None, None, a, None, None, None, None, None, None, 0,
                                        4, 1, 1, 1, 16, 8, 2, 64, 64, 4, 1, 1, 1.0, 0, 0.0, None)
    assert rc == _lib.RPA_ERR_INVALID_ARGUMENT and b"kv_scales" in lib.rpa_last_error()  # scales with 16-bit pages
    rc = lib.rpa_ragged_paged_attention(None, None, None, None, None, None, None, None, None, None, 0,
                                        4, 1, 1, 1, 16, 8, 2, 96, 64, 4, 1, 1, 1.0, 0, 0.0, None)
    assert rc == _lib.RPA_ERR_INVALID_ARGUMENT and b"Dp" in lib.rpa_last_error()  # stored rows narrower than the head
    with pytest.raises(_lib.RpaError):
        _lib.check(rc)
    # the block tables of one call may address at most 2^31 - 1 tokens (S * M * page_size): refused before any device work
    rc = lib.rpa_ragged_paged_attention(None, None, None, None, None, None, None, None, None, None, 0,
                                        4, 4096, 8192, 1 << 20, 64, 8, 2, 64, 64, 4, 1, 1, 1.0, 0, 0.0, None)
    assert rc == _lib.RPA_ERR_UNSUPPORTED and b"2^31" in lib.rpa_last_error()
    rc = lib.rpa_ragged_paged_attention(None, None, None, None, None, None, None, None, None, None, 0,
                                        4, 4096, 8191, 1 << 20, 64, 8, 2, 64, 64, 4, 1, 1, 1.0, 0, 0.0, None)
    assert rc == _lib.RPA_ERR_INVALID_ARGUMENT and b"null pointer" in lib.rpa_last_error()  # one page less per row: the sizes pass
    # int8 pages are always scaled; fp8 pages may hold bare codes (the reference's cast-only cache)
    rc = lib.rpa_ragged_paged_attention(None, None, None, None, None, None, None, None, None, None, 0,
                                        4, 1, 1, 1, 16, 8, 2, 64, 64, 4, 1, 3, 1.0, 0, 0.0, None)
    assert rc == _lib.RPA_ERR_INVALID_ARGUMENT and b"int8 KV pages need kv_scales" in lib.rpa_last_error()
    rc = lib.rpa_ragged_paged_attention(None, None, None, None, None, None, None, None, None, None, 0,
                                        4, 1, 1, 1, 16, 8, 2, 64, 64, 4, 1, 2, 1.0, 0, 0.0, None)
    assert rc == _lib.RPA_ERR_INVALID_ARGUMENT and b"null pointer" in lib.rpa_last_error()
    # pointers are checked for null and alignment before anything is launched (the values below are never dereferenced)
    a = 0x7000_0000_0000
    rc = lib.rpa_ragged_paged_attention(None, a + 8, a, None, a, a, a, a, a, a, 1 << 20,
                                        4, 1, 1, 1, 16, 8, 2, 64, 64, 4, 1, 1, 1.0, 0, 0.0, None)
    assert rc == _lib.RPA_ERR_INVALID_ARGUMENT and b"16-byte aligned" in lib.rpa_last_error()
    rc = lib.rpa_ragged_paged_attention(None, a, a, None, a, a, a, a, a, a, 1 << 20,
                                        4, 1, 1, 1, 16, 8, 2, 64, 64, 4, 1, 1, 1.0, 0, 0.0, a + 2)
    assert rc == _lib.RPA_ERR_INVALID_ARGUMENT and b"softmax_aux" in lib.rpa_last_error()
    rc = lib.rpa_ragged_paged_attention_v3(None, a, None, a, a, a, a, a, a, a, a, 1 << 20,
                                           4, 1, 1, 1, 16, 8, 2, 64, 64, 4, 1, 1, 1.0, 0, 0.0, None)
    assert rc == _lib.RPA_ERR_INVALID_ARGUMENT and b"null key" in lib.rpa_last_error()
    assert lib.rpa_page_scatter_slices(None, None, None, None, None, 0, 0, 0, 4, 16, 0) == 0  # empty input is a no-op
    assert lib.rpa_page_scatter_slices(None, None, None, None, None, 4, 4, 64, 0, 16, 0) == _lib.RPA_ERR_INVALID_ARGUMENT
    n = lib.rpa_attention_workspace_bytes(256, 256, 128, 64, 32, 8, 128, 1, 1)
    assert n > 2 * 256 * 32 * 130 * 4
    # the read probe reads nothing and launches nothing on bad arguments
    assert lib.rpa_read_probe(None, None, 1 << 30, 256, 8, None) == 0 and b"rpa_read_probe" in lib.rpa_last_error()
    assert lib.rpa_read_probe(None, a, 1 << 30, 256, 3, a) == 0  # 2 / 4 / 8 / 16 / 32 KiB in flight per wave
    assert lib.rpa_read_probe(None, a, 1 << 30, 0, 8, a) == 0
    assert lib.rpa_read_probe(None, a, 4096, 256, 8, a) == 0  # less than one round of loads per wave
    assert lib.rpa_read_probe_paged(None, None, 1 << 30, 256, 8, 64, 1, None) == 0 and b"rpa_read_probe_paged" in lib.rpa_last_error()
    assert lib.rpa_read_probe_paged(None, a, 1 << 30, 256, 4, 64, 1, a) == 0  # a wave's eighth of a 64 KiB chunk is 8 KiB
    assert lib.rpa_read_probe_paged(None, a, 1 << 30, 256, 8, 60, 0, a) == 0  # chunk_kib a multiple of 8
    assert lib.rpa_read_probe_paged(None, a, 1 << 30, 256, 8, 64, 3, a) == 0  # split 0..2
    prev = _lib.set_tunable("max_splits", 4)
    assert lib.rpa_attention_workspace_bytes(256, 256, 128, 64, 32, 8, 128, 1, 1) < n
    _lib.set_tunable("max_splits", prev)
    assert _lib.set_tunable("no_such_knob", 1) == -1
    assert lib.rpa_mfma_probe(None, 1, 1, 2, 1, 100, None, None) == 0.0 and b"rpa_mfma_probe" in lib.rpa_last_error()
    assert lib.rpa_mfma_probe(None, 1, 1, 3, 1, 100, a, a) == 0.0  # 1, 2 or 4 MFMAs per operand
    assert lib.rpa_issue_probe(None, 1, 1, 6, 100, None, None, None) == 0 and b"rpa_issue_probe" in lib.rpa_last_error()
    assert lib.rpa_issue_probe(None, 1, 3, 6, 100, a, a, a) == 0  # 0, 1, 2 or 4 instructions beside the MFMA
    assert lib.rpa_issue_probe(None, 10, 1, 6, 100, a, a, a) == 0  # kinds 0..9


def test_workspace_sizing_asks_for_page_copies_only_where_a_call_could_use_them():
    """8-bit pages: the sizing call adds room for bf16 copies of prompt chunks' pages -- for the sequences that can have
    large rows, M pages each -- and nothing for a pure-decode bucket, 16-bit pages, head sizes the kernel on the copies
    does not serve, pages that are not a multiple of 64 tokens, or with the copies switched off."""
    lib = _lib.load()
    f = lib.rpa_attention_workspace_bytes  # (T, S, M, page_size, Hq, Hkv, D, q_dtype, kv_dtype)
    BF16, FP8, INT8 = 1, 2, 3

    def room(*shape):  # what the copies add: the figure with them less the figure with them switched off
        with_copies = f(*shape)
        prev = _lib.set_tunable("prefill_wide", 0)
        try:
            return with_copies - f(*shape)
        finally:
            _lib.set_tunable("prefill_wide", prev)

    page16 = 64 * 2 * 8 * 128 * 2
    for kv in (FP8, INT8):
        assert 4 * 256 * page16 <= room(8192, 4, 256, 64, 40, 8, 128, BF16, kv) < 4 * 256 * page16 + (1 << 16)  # 4 sequences x 256 pages
        assert room(256, 256, 128, 64, 40, 8, 128, BF16, kv) == 0   # 1 280 rows per KV head in all: a pure-decode bucket
        assert room(8192, 4, 256, 32, 40, 8, 128, BF16, kv) == 0   # 32-token pages
        assert room(8192, 4, 256, 64, 8, 8, 64, BF16, kv) == 0     # head size 64
        assert room(8192, 4, 256, 64, 16, 8, 256, BF16, kv) >= 4 * 256 * 2 * page16  # head size 256
    assert room(8192, 4, 256, 64, 40, 8, 128, BF16, BF16) == 0
    # many sequences, few tokens: not all of them can have large rows (more than 16 or 32 rows per KV head each)
    assert 0 < room(2048, 512, 16, 64, 32, 8, 128, BF16, INT8) <= (2048 * 4 // 17) * 16 * page16 + (1 << 16) < 512 * 16 * page16
    # capped at 4 GiB
    assert room(65536, 512, 4096, 64, 32, 8, 128, BF16, INT8) <= (4 << 30) + (1 << 16)


def test_product_build_has_no_probes_and_no_stage_knob(tmp_path):
    """The API source compiled without -DRPA_PROBES (what `python -m easydel_amd.build --product` links) neither defines
    the measurement entry points nor knows the knobs that change what a call computes with."""
    import subprocess

    from easydel_amd import build

    obj = tmp_path / "rpa_api_product.o"
    cmd = [build._hipcc(), *build.HIPCC_FLAGS, "-c", str(build.CSRC / "rpa_api.hip"), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    syms = subprocess.run(["nm", "--defined-only", str(obj)], capture_output=True, text=True).stdout
    for name in _lib.PROBE_SIGNATURES:
        assert name not in syms, f"{name} is defined in a product build"
    assert "rpa_ragged_paged_attention_v3" in syms and "rpa_set_tunable" in syms
    strings = subprocess.run(["strings", str(obj)], capture_output=True, text=True).stdout
    assert "force_generic" not in strings and "\nstages\n" not in "\n" + strings + "\n"
    assert "decode_sync" in strings  # the tuning knobs stay


def test_the_pinned_prefill_steps_are_what_the_source_says(tmp_path):
    """The 32x32-tile prefill kernel issues its MFMAs and its tile requests through assembly statements, which the
    compiler neither pads nor sees into; two things it relies on are checked on the generated code.  (1) m0, which a
    half tile's first request sets for the others, is written by nothing but those statements.  (2) Inside the pinned
    loops (the blocks that hold a whole step's MFMAs) there is no scratch-memory access and no wait on the vector-memory
    counter other than the steps' own: either would wait for the tiles in flight."""
    import re
    import subprocess

    from easydel_amd import build

    asm = tmp_path / "x32.s"
    cmd = [build._hipcc(), *build.HIPCC_FLAGS, "-S", "--cuda-device-only", str(build.CSRC / "rpa_attn_prefill_x32.hip"), "-o", str(asm)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    lines = asm.read_text().splitlines()
    in_asm, kernel, block, blocks = False, None, None, {}
    for n, line in enumerate(lines, 1):
        text = line.strip()
        if "#ASMSTART" in text:
            in_asm = True
        elif "#ASMEND" in text:
            in_asm = False
        m = re.match(r"^(_ZN3rpa23attn_prefill_x32_kernel\w+):", line)
        if m:
            kernel = m.group(1)
        m = re.match(r"^(\.LBB\d+_\d+):", line)
        if m and kernel:
            block = (kernel, m.group(1))
            blocks[block] = []
        if not text or text.startswith(";") or text.startswith("."):
            continue
        if not in_asm:
            assert not re.search(r"\bm0\b", text), f"line {n}: the compiler's own code touches m0: {text}"
        if block:
            blocks[block].append((text, in_asm))
    pinned = {b: ins for b, ins in blocks.items() if sum(t.startswith("v_mfma") for t, _ in ins) >= 30}
    bf16 = [b for b in pinned if "ELi1ELb" in b[0]]  # the bf16 instantiations: the benchmark shapes
    assert len(bf16) >= 6, sorted(pinned)  # two pinned steps each at head size 128, 256 and 256 with soft cap
    for b in bf16:
        ins = pinned[b]
        last = max(i for i, (t, _) in enumerate(ins) if t.startswith("v_mfma"))
        first = min(i for i, (t, _) in enumerate(ins) if t.startswith("v_mfma"))
        for t, from_asm in ins[first:last + 1]:
            assert not t.startswith("scratch_"), f"{b}: scratch access inside a pinned step: {t}"
            assert from_asm or "vmcnt" not in t, f"{b}: the compiler waits on vector memory inside a pinned step: {t}"


def test_multi_latent_entry_points_validate_before_any_device_work():
    lib = _lib.load()
    a = 0x7000_0000_0000
    args = dict(T=4, S=2, M=8, P=16, pg=64, Hq=16, rank=512, rope=64, row=640, qd=1, kd=1)

    def call(qn=a, qp=a, kv=None, pe=None, pages=a, ctx=a, bt=a, qsl=a, dist=a, out=a, ws=a, ws_bytes=1 << 24, aux=None, **over):
        v = dict(args, **over)
        return lib.rpa_mla_ragged_paged_attention(None, qn, qp, kv, pe, pages, ctx, bt, qsl, dist, out, ws, ws_bytes, v["T"], v["S"],
                                                  v["M"], v["P"], v["pg"], v["Hq"], v["rank"], v["rope"], v["row"], v["qd"], v["kd"],
                                                  0.07, 0, 0.0, aux)

    assert call(row=568) == _lib.RPA_ERR_INVALID_ARGUMENT and b"row_elems" in lib.rpa_last_error()
    assert call(rank=1024, row=2048) == _lib.RPA_ERR_UNSUPPORTED and b"kv_lora_rank" in lib.rpa_last_error()
    assert call(kd=3) == _lib.RPA_ERR_UNSUPPORTED and b"kv_dtype" in lib.rpa_last_error()  # int8: the latent cache has no scales
    assert call(dist=None) == _lib.RPA_ERR_INVALID_ARGUMENT and b"distribution" in lib.rpa_last_error()
    assert call(qn=None) == _lib.RPA_ERR_INVALID_ARGUMENT and b"null pointer" in lib.rpa_last_error()
    assert call(kv=a, pe=None) == _lib.RPA_ERR_INVALID_ARGUMENT and b"keys_pe" in lib.rpa_last_error()
    assert call(out=a + 8) == _lib.RPA_ERR_INVALID_ARGUMENT and b"16-byte aligned" in lib.rpa_last_error()
    assert call(ws_bytes=64) == _lib.RPA_ERR_WORKSPACE and b"workspace" in lib.rpa_last_error()
    assert call(T=0) == 0  # an empty batch is a no-op
    n = lib.rpa_mla_workspace_bytes(256, 256, 128, 64, 128, 512, 1, 1)
    assert n > 256 * 128 * 514 * 4  # at least one chunk's partial rows when the shapes ask for a split
    assert lib.rpa_mla_page_scatter(None, a, a, a, a, a, a, a, 4, 2, 8, 16, 64, 512, 64, 640, 3) == _lib.RPA_ERR_UNSUPPORTED
    assert lib.rpa_mla_page_scatter(None, None, a, a, a, a, a, a, 4, 2, 8, 16, 64, 512, 64, 640, 2) == _lib.RPA_ERR_INVALID_ARGUMENT
