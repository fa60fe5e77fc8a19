"""The GGUF parser (csk_gguf_*) against the reference's own readers.

* On any box: the committed checkpoints tests/golden/moe_block*.gguf must parse to the
  table tests/golden/gguf_table.json, which make_gguf_golden.py wrote from the reference's
  gguf_loader / gguf_multi_loader (src/gguf/gguf_loader.cpp:383-518,
  src/gguf/gguf_multi_loader.cpp:25-76) compiled as they lie.
* Where oracle/_ref/libref_gguf.so is present: every kind of file the writer produces at
  alignment 32 (the reference hard-codes it) is parsed by both and compared field by field.
"""
import json
import os

import numpy as np
import pytest

from coalsack_amd import capi, synth
from coalsack_amd import gguf_writer as gw

GOLD = os.path.join(os.path.dirname(__file__), "golden")
REF_SO = os.path.join(os.path.dirname(GOLD), "..", "oracle", "_ref", "libref_gguf.so")


def _same_as_table(g, table, sharded):
    assert sorted(g.tensor_names()) == sorted(table["tensors"])
    for name, want in table["tensors"].items():
        got = g.tensor_info(name)
        assert (got["type"], got["dims"], got["offset"], got["nbytes"]) == \
               (want["type"], want["dims"], want["offset"], want["nbytes"]), name
        assert g.tensor_shard(name) == want["shard"], name
    for key, want in table["u32"].items():
        if want is None:
            with pytest.raises(capi.CskError):
                g.get_u32(key)
        else:
            assert g.get_u32(key) == want, key
    for key, want in table["str"].items():
        if want is None:
            with pytest.raises(capi.CskError):
                g.get_str(key)
        else:
            assert g.get_str(key) == want, key


def test_golden_checkpoint_parses_to_the_reference_table():
    lib = capi.Library()
    table = json.load(open(os.path.join(GOLD, "gguf_table.json")))
    with lib.gguf(os.path.join(GOLD, "moe_block.gguf")) as g:
        _same_as_table(g, table["single"], False)
    with lib.gguf([os.path.join(GOLD, "moe_block.gguf"), os.path.join(GOLD, "moe_block_shard2.gguf")]) as g:
        _same_as_table(g, table["sharded"], True)
        assert g.tensor_shard("blk.1.ffn_up_exps.weight") == 1 and g.tensor_shard("token_embd.weight") == 0
    # the same name in two shards is refused (gguf_multi_loader.cpp:64-67)
    with pytest.raises(capi.CskError, match="Duplicate tensor name"):
        lib.gguf([os.path.join(GOLD, "moe_block.gguf"), os.path.join(GOLD, "moe_block.gguf")])


def _writer_files(tmp_path):
    """One of each kind of file the writer is used for, alignment 32."""
    rng = np.random.default_rng(3)
    L = synth.LayerInputs(6, 2, 64, 96, seed=5, with_norm=True)
    meta = [("general.architecture", gw.STR, "gpt-oss"), ("gpt-oss.expert_count", gw.U32, 6),
            ("gpt-oss.expert_used_count", gw.U32, 2), ("some.i8", gw.I8, -3), ("some.f64", gw.F64, 2.5),
            ("some.bool", gw.BOOL, 1), ("tokenizer.ggml.tokens", gw.ARR, (gw.STR, ["a", "bc", "", "def"])),
            ("tokenizer.ggml.scores", gw.ARR, (gw.F32, [0.5, -1.0, 2.0])),
            ("tokenizer.ggml.token_type", gw.ARR, (gw.I32, [1, 2, 3, 4, 5]))]
    out = []
    p = str(tmp_path / "mx.gguf")
    gw.write_gguf(p, meta, [("token_embd.weight", gw.GGML_F16, [64, 10], np.zeros(640, np.float16).tobytes())]
                  + gw.moe_block_tensors(L, 0) + gw.moe_block_tensors(L, 1, bias=False))
    out.append(p)
    L2 = synth.LayerInputs(3, 2, 256, 256, seed=6, with_norm=True)
    f16w = [[rng.normal(0, 0.1, s).astype(np.float16) for s in ((256, 256), (256, 256), (256, 256))] for _ in range(3)]
    p = str(tmp_path / "f16.gguf")
    gw.write_gguf(p, [("general.architecture", gw.STR, "llama4"), ("llama4.expert_count", gw.U32, 3),
                      ("llama4.expert_used_count", gw.U32, 2)],
                  gw.moe_block_tensors(L2, 0, f16_weights=f16w, norm_name="ffn_norm.weight"))
    out.append(p)
    q4 = [rng.integers(0, 256, 256 * 256 // 256 * 144, dtype=np.uint8).tobytes() for _ in range(3)]
    q6 = [rng.integers(0, 256, 256 * 256 // 256 * 210, dtype=np.uint8).tobytes() for _ in range(3)]
    p = str(tmp_path / "kq.gguf")
    gw.write_gguf(p, [("general.architecture", gw.STR, "llama4"), ("llama4.expert_count", gw.U32, 3)],
                  gw.moe_block_tensors(L2, 0, raw_weights=[(12, q4), (14, q6), (12, q4)], norm_name="ffn_norm.weight"))
    out.append(p)
    return out


@pytest.mark.skipif(not os.path.exists(REF_SO), reason="oracle/_ref/libref_gguf.so not built (no reference tree)")
def test_writer_files_parse_like_the_reference_loader(tmp_path):
    from oracle.binding import RefGguf
    lib = capi.Library()
    paths = _writer_files(tmp_path)
    for case in [[p] for p in paths] + [paths[:2]]:
        # (the two-file case pairs files with disjoint tensor names? no: both hold blk.0 -- refused by both)
        ref = RefGguf(case)
        if len(case) > 1:
            assert not ref.loaded
            with pytest.raises(capi.CskError, match="Duplicate tensor name"):
                lib.gguf(case)
            continue
        assert ref.loaded
        with lib.gguf(case[0]) as g:
            names = g.tensor_names()
            assert sorted(names) == sorted(ref.tensor_names())
            for name in names:
                got, want = g.tensor_info(name), ref.tensor_info(name)
                assert (got["type"], got["dims"], got["offset"], got["nbytes"]) == \
                       (want["type"], want["dims"], want["offset"], want["nbytes"]), (case, name)
            for key in ("gpt-oss.expert_count", "gpt-oss.expert_used_count", "llama4.expert_count", "no.such.key"):
                want = ref.get_u32(key)
                if want is None:
                    with pytest.raises(capi.CskError):
                        g.get_u32(key)
                else:
                    assert g.get_u32(key) == want
            assert g.get_str("general.architecture") == ref.get_str("general.architecture")
        ref.close()


def test_damaged_tables_are_refused_not_followed(tmp_path):
    """Offsets and dimensions whose sums or products wrap 64 bits must end in an error, never
    in a pointer outside the file."""
    import struct
    lib = capi.Library()
    L = synth.LayerInputs(2, 1, 64, 96, seed=5)
    p = str(tmp_path / "ok.gguf")
    gw.write_gguf(p, [("general.architecture", gw.STR, "gpt-oss")], gw.moe_block_tensors(L, 0, norm=False))
    raw = bytearray(open(p, "rb").read())
    name = b"blk.0.ffn_up_exps.weight"
    at = raw.index(name) + len(name)          # n_dims (u32), 3 dims (u64), type (u32), offset (u64)
    off_field = at + 4 + 3 * 8 + 4
    for bad_off in (2**64 - 32, 2**64 - 1, 2**63, len(raw)):
        b = bytearray(raw)
        b[off_field:off_field + 8] = struct.pack("<Q", bad_off)
        q = tmp_path / "bad_off.gguf"
        q.write_bytes(b)
        with pytest.raises(capi.CskError, match="past the end of the file"):
            lib.gguf(str(q))
    for bad_dims in ((2**32, 2**32, 2**32), (2**63, 4, 1), (2**62, 2**62, 17)):
        b = bytearray(raw)
        b[at + 4:at + 4 + 24] = struct.pack("<QQQ", *bad_dims)
        q = tmp_path / "bad_dims.gguf"
        q.write_bytes(b)
        with pytest.raises(capi.CskError, match="overflows|past the end of the file"):
            lib.gguf(str(q))
