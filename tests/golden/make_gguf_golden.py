"""Writes tests/golden/moe_block.gguf (+ its second shard) and tests/golden/gguf_table.json:
small synthetic checkpoints written by coalsack_amd/gguf_writer.py, and what the reference's
own readers (gguf_loader / gguf_multi_loader, compiled from the reference tree into
oracle/_ref/libref_gguf.so by oracle/Makefile) report for them -- version, tensor names,
types, dims, absolute offsets, sizes, shard indices and the metadata the MoE path reads.

Run in a container that has the reference tree:  python tests/golden/make_gguf_golden.py
"""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from coalsack_amd import gguf_writer as gw, synth  # noqa: E402
from oracle.binding import RefGguf  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
KEYS_U32 = ["gpt-oss.expert_count", "gpt-oss.expert_used_count", "gpt-oss.block_count", "some.u8"]
KEYS_STR = ["general.architecture", "general.name"]


def files():
    L = synth.LayerInputs(4, 2, 64, 96, seed=11, with_norm=True)
    meta = [("general.architecture", gw.STR, "gpt-oss"), ("general.name", gw.STR, "golden"),
            ("gpt-oss.expert_count", gw.U32, 4), ("gpt-oss.expert_used_count", gw.U32, 2),
            ("gpt-oss.block_count", gw.U32, 2), ("some.u8", gw.U8, 7), ("some.f32", gw.F32, 1.5),
            ("tokenizer.ggml.tokens", gw.ARR, (gw.STR, ["a", "bc", ""])),
            ("tokenizer.ggml.scores", gw.ARR, (gw.F32, [0.5, -1.0]))]
    t0 = [("token_embd.weight", gw.GGML_F16, [64, 5], np.arange(320, dtype=np.float16).tobytes())]
    t0 += gw.moe_block_tensors(L, 0)
    t1 = gw.moe_block_tensors(L, 1, bias=False)
    meta1 = [("general.architecture", gw.STR, "gpt-oss"), ("split.no", gw.U32, 1)]
    return [("moe_block.gguf", meta, t0), ("moe_block_shard2.gguf", meta1, t1)]


def table(ref):
    out = dict(version=ref.version(), tensors={})
    for name in sorted(ref.tensor_names()):
        out["tensors"][name] = ref.tensor_info(name)
    out["u32"] = {k: ref.get_u32(k) for k in KEYS_U32 + ["gpt-oss.nope"]}
    out["str"] = {k: ref.get_str(k) for k in KEYS_STR + ["general.nope"]}
    return out


def main():
    paths = []
    for name, meta, tensors in files():
        p = os.path.join(HERE, name)
        gw.write_gguf(p, meta, tensors)
        paths.append(p)
    one = RefGguf(paths[0])
    both = RefGguf(paths)
    assert one.loaded and both.loaded
    json.dump(dict(single=table(one), sharded=table(both)), open(os.path.join(HERE, "gguf_table.json"), "w"),
              indent=1, sort_keys=True)
    print("wrote", [os.path.basename(p) for p in paths], "and gguf_table.json")


if __name__ == "__main__":
    main()
