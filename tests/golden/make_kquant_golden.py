"""Writes tests/golden/kquant_codec.npz from the reference's own K-quant codecs and
fp32 -> fp16 conversion (oracle/_ref/libref_mxfp4.so, built by oracle/Makefile from
include/coalsack/gguf/gguf_dequant.h of the reference tree, composed the way
src/llm/moe_weight_provider.cpp:17-33 widens Q4_K / Q6_K expert slices to fp16).

Contents: `q4_blocks` (48 x 144 bytes) / `q6_blocks` (48 x 210 bytes) = seeded random
super-blocks whose fp16 scale fields are finite; `q4_f32`, `q6_f32` = their fp32
dequantisation (uint32 bit patterns); `q4_f16`, `q6_f16` = the fp16 halves the weight
provider would hand to the expert node; `cvt_in` / `cvt_out` = fp32 bit patterns covering
every exponent, the rounding boundaries and the subnormal range, and their conversion.

Run in a container that has the reference tree:  python tests/golden/make_kquant_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle.binding import RefCodec  # noqa: E402


def finite_halves(rng, n, lo=-12, hi=-3):
    """n fp16 bit patterns of magnitude 2^lo .. 2^hi, either sign."""
    v = np.ldexp(rng.uniform(1.0, 2.0, n), rng.integers(lo, hi, n)) * rng.choice([-1.0, 1.0], n)
    return v.astype(np.float16).view(np.uint16)


def random_blocks(rng, kind, n):
    size = 144 if kind == "q4_k" else 210
    b = rng.integers(0, 256, (n, size), dtype=np.uint8)
    if kind == "q4_k":
        b[:, 0:2] = finite_halves(rng, n).view(np.uint8).reshape(n, 2)
        b[:, 2:4] = finite_halves(rng, n).view(np.uint8).reshape(n, 2)
    else:
        b[:, 208:210] = finite_halves(rng, n).view(np.uint8).reshape(n, 2)
    return b


def conversion_inputs(rng):
    pats = []
    for e in range(256):  # every fp32 exponent, mantissas at and around the fp16 rounding boundaries
        for m in (0, 1, 0x0FFF, 0x1000, 0x1001, 0x1FFF, 0x2000, 0x3000, 0x7FE000, 0x7FFFFF):
            for s in (0, 1):
                pats.append((s << 31) | (e << 23) | m)
    pats = np.array(pats, np.uint32)
    pats = pats[np.isfinite(pats.view(np.float32))]
    rnd = rng.integers(0, 2 ** 32, 4096, dtype=np.uint64).astype(np.uint32)
    rnd = rnd[np.isfinite(rnd.view(np.float32))]
    return np.concatenate([pats, rnd])


def main():
    ref = RefCodec()
    assert ref.has_kquant
    rng = np.random.default_rng(20240711)
    out = {}
    for kind, tag in (("q4_k", "q4"), ("q6_k", "q6")):
        b = random_blocks(rng, kind, 48)
        out[tag + "_blocks"] = b
        out[tag + "_f32"] = ref.dequant_kquant(kind, b.reshape(-1), 48 * 256).view(np.uint32)
        out[tag + "_f16"] = ref.kquant_to_fp16(kind, b.reshape(-1), 48 * 256)
    cin = conversion_inputs(rng)
    out["cvt_in"] = cin
    out["cvt_out"] = ref.fp32_to_fp16(cin.view(np.float32))
    np.savez_compressed(os.path.join(os.path.dirname(__file__), "kquant_codec.npz"), **out)
    print("wrote kquant_codec.npz", {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
