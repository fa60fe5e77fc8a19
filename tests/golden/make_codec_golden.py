"""Writes tests/golden/mxfp4_codec.npz from the reference's own codec
(oracle/_ref/libref_mxfp4.so, built by oracle/Makefile from
include/coalsack/gguf/gguf_dequant.h of the reference tree).

Contents: `scales` = e8m0_to_fp32_half(b) for b = 0..255 (as uint32 bit
patterns); `blocks` = 64 seeded random 17-byte blocks plus 256 blocks that
sweep every scale byte with the 16 codes in both nibble positions; `values` =
dequantize_block_mxfp4 of those blocks (uint32 bit patterns).

Run in a container that has the reference tree:  python tests/golden/make_codec_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle.binding import RefCodec  # noqa: E402


def main():
    ref = RefCodec()
    scales = np.array([ref.e8m0(b) for b in range(256)], np.float32)
    rng = np.random.default_rng(20240611)
    rand = rng.integers(0, 256, (64, 17), dtype=np.uint8)
    sweep = np.empty((256, 17), np.uint8)
    for b in range(256):
        sweep[b, 0] = b
        # byte j: low nibble = code j, high nibble = code 15 - j  (all 16 codes in both positions)
        sweep[b, 1:] = [(j & 15) | (((15 - j) & 15) << 4) for j in range(16)]
    blocks = np.concatenate([rand, sweep])
    values = ref.dequant(blocks.reshape(-1), blocks.shape[0] * 32)
    np.savez_compressed(os.path.join(os.path.dirname(__file__), "mxfp4_codec.npz"),
                        scales=scales.view(np.uint32), blocks=blocks, values=values.view(np.uint32))
    print("wrote mxfp4_codec.npz", blocks.shape, values.shape)


if __name__ == "__main__":
    main()
