"""Pins the oracle's K-quant codecs and fp32 -> fp16 conversion (oracle/moe_oracle.c:
orc_dequant_q4_k, orc_dequant_q6_k, orc_fp32_to_fp16, orc_q4k_to_fp16, orc_q6k_to_fp16)
against the committed fixture written from the reference's own header, against that build
itself where it is present, and against closed forms."""
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(__file__), "golden", "kquant_codec.npz")


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD)


@pytest.mark.parametrize("kind,tag", [("q4_k", "q4"), ("q6_k", "q6")])
def test_codecs_match_reference_fixture(oracle, gold, kind, tag):
    b = gold[tag + "_blocks"]
    k = b.shape[0] * 256
    assert np.array_equal(oracle.dequant_kquant(kind, b.reshape(-1), k).view(np.uint32), gold[tag + "_f32"])
    assert np.array_equal(oracle.kquant_to_fp16(kind, b.reshape(-1), k), gold[tag + "_f16"])


def test_conversion_matches_reference_fixture(oracle, gold):
    got = oracle.fp32_to_fp16(gold["cvt_in"].view(np.float32))
    assert np.array_equal(got, gold["cvt_out"])


def test_conversion_truncates(oracle):
    """The reference's build has no F16C: the conversion drops the low 13 mantissa bits
    instead of rounding (gguf_dequant.h:463-487), so it never exceeds the magnitude of its
    input and differs from round-to-nearest on about half of all inputs."""
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(2000) * 0.1).astype(np.float32)
    x = x[np.abs(x) > 1e-3]  # fp16-normal range
    h = oracle.fp32_to_fp16(x).view(np.float16).astype(np.float32)
    assert np.all(np.abs(h) <= np.abs(x))
    assert np.all(np.abs(x) - np.abs(h) < np.abs(x) * 2.0 ** -10)
    rne = x.astype(np.float16).astype(np.float32)
    assert 0.3 < np.mean(h != rne) < 0.7
    assert oracle.fp32_to_fp16(np.array([1e6], np.float32))[0] == 0x7C00
    assert oracle.fp32_to_fp16(np.array([-1e-9], np.float32))[0] == 0x8000


def test_q4_k_closed_form(oracle):
    """One super-block by hand: d = 0.5, dmin = 0.25, sub-block j has scale j + 1 and min j,
    every nibble of sub-block j equals j: value = 0.5 (j + 1) j - 0.25 j."""
    b = np.zeros(144, np.uint8)
    b[0:2] = np.array([0.5], np.float16).view(np.uint8)
    b[2:4] = np.array([0.25], np.float16).view(np.uint8)
    sc = [j + 1 for j in range(8)]
    mn = [j for j in range(8)]
    for j in range(4):  # gguf_dequant.h:172-186: 6-bit fields, the upper four split over two bytes
        b[4 + j] = sc[j] | ((sc[j + 4] >> 4) << 6)
        b[8 + j] = mn[j] | ((mn[j + 4] >> 4) << 6)
        b[12 + j] = (sc[j + 4] & 0xF) | ((mn[j + 4] & 0xF) << 4)
    for pair in range(4):
        b[16 + 32 * pair:16 + 32 * pair + 32] = (2 * pair) | ((2 * pair + 1) << 4)
    got = oracle.dequant_kquant("q4_k", b, 256).reshape(8, 32)
    for j in range(8):
        assert np.all(got[j] == 0.5 * (j + 1) * j - 0.25 * j), j


def test_q6_k_closed_form(oracle):
    """d = 0.125, scale of group g (16 values) = g - 8, all quants = 5 (stored 37):
    value = 0.125 (g - 8) 5."""
    b = np.zeros(210, np.uint8)
    b[0:128] = (37 & 0xF) | ((37 & 0xF) << 4)
    b[128:192] = 0b10101010  # high bit pairs = 2 -> 32 + 5
    b[192:208] = np.arange(-8, 8, dtype=np.int8).view(np.uint8)
    b[208:210] = np.array([0.125], np.float16).view(np.uint8)
    got = oracle.dequant_kquant("q6_k", b, 256).reshape(16, 16)
    for g in range(16):
        assert np.all(got[g] == 0.125 * (g - 8) * 5), g


def test_matches_reference_build_when_present(oracle):
    from oracle.binding import RefCodec
    try:
        ref = RefCodec()
    except (FileNotFoundError, OSError):
        pytest.skip("oracle/_ref is only built where the reference tree is present")
    if not ref.has_kquant:
        pytest.skip("oracle/_ref predates the K-quant entry points")
    from tests.golden.make_kquant_golden import random_blocks
    rng = np.random.default_rng(77)
    for kind in ("q4_k", "q6_k"):
        b = random_blocks(rng, kind, 200).reshape(-1)
        assert np.array_equal(oracle.dequant_kquant(kind, b, 200 * 256).view(np.uint32),
                              ref.dequant_kquant(kind, b, 200 * 256).view(np.uint32))
        assert np.array_equal(oracle.kquant_to_fp16(kind, b, 200 * 256), ref.kquant_to_fp16(kind, b, 200 * 256))
