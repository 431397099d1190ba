"""Pins the oracle's number-format codecs against torch's CPU casts (independent implementations)."""

import numpy as np
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
