"""Pins of the NF4 oracle.  CPU only."""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import quant_oracle as qo  # noqa: E402


def test_levels():
    L = qo.NF4_LEVELS
    assert L[0] == -1.0 and L[15] == 1.0 and L[7] == 0.0
    assert np.all(np.diff(L) > 0)
    # the positive side has one more level than the negative side (asymmetric code)
    assert (L > 0).sum() == 8 and (L < 0).sum() == 7


def test_hand_packed_block():
    # block of 64: absmax 2.0; elements 2.0 -> code 15, -2.0 -> 0, 0 -> 7, 1.0 -> 0.5 -> nearest level 0.4407 (12; 0.5626 is 0.0033 further)
    x = np.zeros(64, dtype=np.float32)
    x[0], x[1], x[2], x[3] = 2.0, -2.0, 0.0, 1.0
    packed, absmax = qo.quantize(x, 64)
    assert absmax.tolist() == [2.0]
    assert packed[0] == (15 << 4) | 0 and packed[1] == (7 << 4) | 12 and packed[2] == (7 << 4) | 7
    y = qo.dequantize(packed, absmax, 64)
    assert y[0] == 2.0 and y[1] == -2.0 and y[2] == 0.0
    assert y[3] == np.float32(0.44070982933044434) * np.float32(2.0)


def test_round_trip_bound():
    g = np.random.default_rng(0)
    x = g.standard_normal(64 * 50).astype(np.float32)
    packed, absmax = qo.quantize(x, 64)
    y = qo.dequantize(packed, absmax, 64)
    half_gap = np.diff(qo.NF4_LEVELS).max() / 2
    err = np.abs(x - y).reshape(-1, 64) / absmax[:, None]
    assert err.max() <= half_gap + 1e-6
    # the element that sets the block maximum is reproduced exactly
    idx = np.abs(x.reshape(-1, 64)).argmax(axis=1)
    assert np.array_equal(y.reshape(-1, 64)[np.arange(50), idx], x.reshape(-1, 64)[np.arange(50), idx])


def test_nested_absmax_and_bf16():
    code2 = np.linspace(-1, 1, 256).astype(np.float32)
    q = np.array([0, 255, 128, 3] * 128, dtype=np.uint8)          # 512 blocks -> 2 scales
    a2 = np.array([2.0, 4.0], dtype=np.float32)
    out = qo.nested_absmax(q, code2, a2, 0.5)
    assert out[0] == -2.0 + 0.5 and out[1] == 2.0 + 0.5 and out[256] == -4.0 + 0.5
    assert qo.to_bf16_bits(np.array([1.0, -2.0, 1.00390625], dtype=np.float32)).tolist() == [0x3F80, 0xC000, 0x3F80]
    assert qo.to_bf16_bits(np.array([1.01171875], dtype=np.float32)).tolist() == [0x3F82]  # tie -> even
