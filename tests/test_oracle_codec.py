"""Pins the oracle's MXFP4 codec (oracle/moe_oracle.c) against the reference's
own codec (oracle/_ref when built, else the committed fixture it produced), the
reference's known answers and the closed form."""
import math
import os

import numpy as np
import pytest

LUT = np.array([0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12], np.float64)
GOLD = os.path.join(os.path.dirname(__file__), "golden", "mxfp4_codec.npz")


def test_e8m0_known_answers(oracle):
    # test/test_gguf_dequant.cpp:266-279
    assert oracle.e8m0(127) == 0.5
    assert oracle.e8m0(128) == 1.0
    assert oracle.e8m0(129) == 2.0


def test_e8m0_closed_form_all_bytes(oracle):
    for b in range(256):
        assert oracle.e8m0(b) == math.ldexp(1.0, b - 128), b  # 2^-128, 2^-127 are fp32 denormals


def test_dequant_zero_block_known_answer(oracle):
    # test/test_gguf_dequant.cpp:244-263
    blk = np.zeros(17, np.uint8)
    blk[0] = 128
    assert np.all(oracle.dequant(blk, 32) == 0.0)


def test_dequant_closed_form_exhaustive(oracle):
    """All 256 scale bytes x 16 codes x both nibble positions against
    lut[c] * 2^(e-128) evaluated in float64 (exact)."""
    for e in range(256):
        blk = np.zeros(17, np.uint8)
        blk[0] = e
        lo = np.arange(16)
        hi = (lo * 7 + 3) % 16
        blk[1:] = lo | (hi << 4)
        got = oracle.dequant(blk, 32)
        with np.errstate(over="ignore"):  # 8 * 2^126 and above round to inf in fp32, as in the reference
            want = (np.concatenate([LUT[lo], LUT[hi]]) * math.ldexp(1.0, e - 128)).astype(np.float32)
        assert np.array_equal(got, want), e


def test_nibble_placement(oracle):
    """Low nibble of byte j -> element j, high nibble -> element j + 16
    (gguf_dequant.h:447-453; the bench quantiser packs the same way,
    test/bench_expert_mlp_mxfp4.cpp:68-70)."""
    for j in range(16):
        blk = np.zeros(17, np.uint8)
        blk[0] = 128
        blk[1 + j] = 0x21  # low nibble code 1 (+1), high nibble code 2 (+2)
        out = oracle.dequant(blk, 32)
        want = np.zeros(32, np.float32)
        want[j], want[j + 16] = 1.0, 2.0
        assert np.array_equal(out, want)


def test_against_reference_fixture(oracle):
    g = np.load(GOLD)
    scales = np.array([oracle.e8m0(b) for b in range(256)], np.float32)
    assert np.array_equal(scales.view(np.uint32), g["scales"])
    vals = oracle.dequant(g["blocks"].reshape(-1), g["blocks"].shape[0] * 32)
    assert np.array_equal(vals.view(np.uint32), g["values"])


def test_against_reference_build(oracle):
    """Bit-exact against the reference's header compiled as oracle/_ref (only
    where that library exists: it is built from the reference tree)."""
    from oracle.binding import RefCodec
    try:
        ref = RefCodec()
    except (FileNotFoundError, OSError):
        pytest.skip("oracle/_ref not built here (no reference tree); the committed fixture covers it")
    rng = np.random.default_rng(5)
    blocks = rng.integers(0, 256, (2000, 17), dtype=np.uint8)
    a = oracle.dequant(blocks.reshape(-1), 2000 * 32)
    b = ref.dequant(blocks.reshape(-1), 2000 * 32)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    for x in range(256):
        assert oracle.e8m0(x) == ref.e8m0(x)


def test_synth_generator_layout():
    """Host replay of the device weight generator: scale bytes within the
    configured range and uniform, nibbles uniform over the 16 codes."""
    from coalsack_amd import synth
    b = synth.mxfp4_blocks(7, 3, 5, 1, 64, 2880).reshape(-1, 17)
    assert b.shape == (64 * 90, 17)
    assert b[:, 0].min() == 117 and b[:, 0].max() == 121
    counts = np.bincount(b[:, 0], minlength=122)[117:122] / b.shape[0]
    assert np.all(np.abs(counts - 0.2) < 0.03)
    nib = np.concatenate([(b[:, 1:] & 15).ravel(), (b[:, 1:] >> 4).ravel()])
    freq = np.bincount(nib, minlength=16) / nib.size
    assert np.all(np.abs(freq - 1 / 16) < 0.005)
    # streams differ per expert / matrix / layer
    assert not np.array_equal(b.ravel(), synth.mxfp4_blocks(7, 3, 6, 1, 64, 2880))
    assert not np.array_equal(b.ravel(), synth.mxfp4_blocks(7, 3, 5, 2, 64, 2880))
    assert not np.array_equal(b.ravel(), synth.mxfp4_blocks(7, 4, 5, 1, 64, 2880))
