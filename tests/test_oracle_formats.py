"""Pins the oracle's number-format codecs against torch's CPU casts (independent implementations)."""

import numpy as np
import pytest
import torch

from rpa_testlib import orc


def test_e4m3fn_decode_all_codes_match_torch():
    codes = np.arange(256, dtype=np.uint8)
    want = torch.from_numpy(codes).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    got = orc.e4m3fn_bits_to_f32(codes)
    np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
    np.testing.assert_array_equal(got[~np.isnan(got)], want[~np.isnan(want)])
    assert got[0x7E] == 448.0 and got[0x08] == 2.0 ** -6 and got[0x01] == 2.0 ** -9


def test_e4m3fn_encode_matches_torch_in_range():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 3, np.linspace(-448, 448, 4001, dtype=np.float32),
                        orc.e4m3fn_decode_table()[:127], np.float32([0.0, -0.0, 1e-9, 2 ** -10, 3 * 2 ** -10])])
    got = orc.f32_to_e4m3fn_bits(x)
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    np.testing.assert_array_equal(got, want)
    # round trip on representable values is the identity
    table = orc.e4m3fn_decode_table()
    finite = np.array([c for c in range(256) if not np.isnan(table[c]) and c != 0x80], dtype=np.uint8)
    np.testing.assert_array_equal(orc.f32_to_e4m3fn_bits(table[finite]), finite)


def test_bf16_round_trip_matches_torch():
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(50000).astype(np.float32) * 10, np.float32([0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895e38])])
    got = orc.f32_to_bf16_bits(x)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(orc.bf16_bits_to_f32(got), torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy())


# ---- quantising page write: the scaled 8-bit page format this build defines ------------------------------

def _one_seq(rng, ctx, q_len, pg=16, Hkv=2, D=32, P=12):
    bt = np.arange(1, 1 + -(-ctx // pg), dtype=np.int32)[None]
    bt = np.pad(bt, ((0, 0), (0, 8 - bt.shape[1])))
    k = rng.standard_normal((q_len, Hkv, D)).astype(np.float32)
    v = (3.0 * rng.standard_normal((q_len, Hkv, D))).astype(np.float32)
    return bt, k, v, np.array([ctx], np.int32), np.array([0, q_len], np.int32)


@pytest.mark.parametrize("kv_dtype", [orc.FP8_E4M3, orc.INT8])
def test_quantised_write_of_whole_pages_is_one_shot_quantisation(kv_dtype):
    rng = np.random.default_rng(0)
    pg, Hkv, D, P = 16, 2, 32, 12
    bt, k, v, ctx, qsl = _one_seq(rng, 40, 40)
    stale_codes = rng.integers(0, 255, size=(P, pg, 2 * Hkv, D), dtype=np.uint8)
    stale_scales = np.full((P, 2 * Hkv), 99.0, np.float32)  # a recycled page's scale must not leak into its new owner
    codes, scales = orc.page_scatter_ragged_quantised_ref(k, v, stale_codes, stale_scales, ctx, bt, qsl, [1], kv_dtype=kv_dtype)
    qmax = np.float32(orc.QMAX[kv_dtype])
    for j, (lo, hi) in enumerate([(0, 16), (16, 32), (32, 40)]):
        page = bt[0, j]
        for c in range(2 * Hkv):
            x = (v if c & 1 else k)[lo:hi, c >> 1]
            s = np.float32(np.abs(x).max()) / qmax
            assert scales[page, c] == s
            assert np.array_equal(codes[page, :hi - lo, c], orc.quantise_codes(x / s, kv_dtype))
        assert np.array_equal(codes[page, hi - lo:], stale_codes[page, hi - lo:])  # slots past the context untouched
    untouched = [p for p in range(P) if p not in bt[0, :3]]
    assert np.array_equal(codes[untouched], stale_codes[untouched]) and np.array_equal(scales[untouched], stale_scales[untouched])
    # int8: half a step; fp8: half the spacing of the top binade (32 codes) at most
    for c in range(2 * Hkv):
        x = (v if c & 1 else k)[0:16, c >> 1]
        deq = orc.decode_codes(codes[bt[0, 0], :16, c], kv_dtype) * scales[bt[0, 0], c]
        bound = scales[bt[0, 0], c] * (0.5 if kv_dtype == orc.INT8 else 16.0)
        assert np.abs(deq - x).max() <= bound * (1 + 1e-6)


@pytest.mark.parametrize("kv_dtype", [orc.FP8_E4M3, orc.INT8])
def test_quantised_write_scales_only_grow_and_old_tokens_are_recoded(kv_dtype):
    rng = np.random.default_rng(1)
    pg, Hkv, D, P = 16, 1, 32, 4
    bt = np.array([[2, 3, 0, 0]], np.int32)
    codes = np.zeros((P, pg, 2, D), np.uint8)
    scales = np.zeros((P, 2), np.float32)
    history = []
    prev_scale = np.zeros(2, np.float32)
    for step, gain in enumerate([1.0, 0.2, 5.0, 0.1, 5.0]):
        k = (gain * rng.standard_normal((1, Hkv, D))).astype(np.float32)
        v = (gain * rng.standard_normal((1, Hkv, D))).astype(np.float32)
        history.append((k[0, 0], v[0, 0]))
        before = codes.copy()
        codes, scales = orc.page_scatter_ragged_quantised_ref(k, v, codes, scales, np.array([step + 1], np.int32), bt,
                                                              np.array([0, 1], np.int32), [1], kv_dtype=kv_dtype)
        assert (scales[2] >= prev_scale).all()
        grew = scales[2] > prev_scale
        for c in range(2):
            if not grew[c] and step > 0:  # scale kept: tokens already in the page keep their codes
                assert np.array_equal(codes[2, :step, c], before[2, :step, c])
        prev_scale = scales[2].copy()
    # after all steps every token is within one step of the final scale of its value (two roundings at most: written, re-coded)
    for r, (kk, vv) in enumerate(history):
        for c, x in enumerate((kk, vv)):
            deq = orc.decode_codes(codes[2, r, c], kv_dtype) * scales[2, c]
            bound = scales[2, c] * (1.0 if kv_dtype == orc.INT8 else 32.0)
            assert np.abs(deq - x).max() <= bound * (1 + 1e-6)


def test_quantised_write_places_tokens_like_the_plain_ragged_write():
    rng = np.random.default_rng(2)
    pg, Hkv, D, P = 16, 2, 32, 20
    ctx = np.array([37, 5, 16], np.int32)
    q_lens = np.array([9, 5, 1], np.int32)
    qsl = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    bt = rng.permutation(np.arange(1, P)).astype(np.int32)[:9].reshape(3, 3)
    k = rng.standard_normal((15, Hkv, D)).astype(np.float32) + 10.0  # never zero: every written row changes
    v = rng.standard_normal((15, Hkv, D)).astype(np.float32) + 10.0
    zero_codes = np.zeros((P, pg, 2 * Hkv, D), np.uint8)
    codes, _ = orc.page_scatter_ragged_quantised_ref(k, v, zero_codes, np.zeros((P, 2 * Hkv), np.float32), ctx, bt, qsl, [3], kv_dtype=orc.INT8)
    plain = orc.page_scatter_ragged_ref(k, v, np.zeros((P, pg, 2 * Hkv, D), np.float32), ctx, bt, qsl, [3])
    assert np.array_equal(codes.any(axis=(2, 3)), (plain != 0).any(axis=(2, 3)))


def test_plain_e4m3fn_cast_matches_torch_incl_overflow_to_nan():
    """The cast-only fp8 cache of the reference: round to nearest even, overflow -> NaN (no saturation)."""
    import torch

    rng = np.random.default_rng(5)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * np.float32(40.0),
                        np.array([0.0, -0.0, 447.9, 448.0, 463.9, 464.0, 464.1, 480.0, 1e6, -464.0, -464.1, -1e9, np.inf, -np.inf,
                                  2.0 ** -9, 2.0 ** -10, 1.5 * 2.0 ** -10, 2.0 ** -10 * 1.01], np.float32),
                        orc.e4m3fn_decode_table()[np.arange(256) % 128 != 127]])
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = orc.cast_e4m3fn_ref(x)
    nan_w, nan_g = (want & 0x7F) == 0x7F, (got & 0x7F) == 0x7F
    assert np.array_equal(nan_w, nan_g) and nan_w.sum() == 7
    assert np.array_equal(want[~nan_w], got[~nan_g])
