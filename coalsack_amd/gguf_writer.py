"""Minimal GGUF v3 writer (synthetic checkpoints for the ingest tests and benchmark): metadata of every scalar type,
string and scalar arrays, tensors with explicit ggml type ids.  Follows the
file layout the reference's reader parses (src/gguf/gguf_loader.cpp:383-518)."""
import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STR, ARR, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B",
        U64: "<Q", I64: "<q", F64: "<d"}
GGML_F32, GGML_F16, GGML_MXFP4 = 0, 1, 39


def _s(text):
    b = text.encode()
    return struct.pack("<Q", len(b)) + b


def _value(vtype, v):
    if vtype == STR:
        return _s(v)
    if vtype == ARR:
        etype, items = v
        out = struct.pack("<IQ", etype, len(items))
        for it in items:
            out += _value(etype, it)
        return out
    return struct.pack(_FMT[vtype], v)


def write_gguf(path, metadata, tensors, alignment=32, version=3):
    """metadata: list of (key, type, value); tensors: list of (name, ggml_type, dims in
    file order (fastest first), bytes-like data)."""
    head = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(metadata))
    for key, vtype, v in metadata:
        head += _s(key) + struct.pack("<I", vtype) + _value(vtype, v)
    offsets, pos = [], 0
    for _, _, _, data in tensors:
        offsets.append(pos)
        pos += (len(data) + alignment - 1) // alignment * alignment
    for (name, gtype, dims, _), off in zip(tensors, offsets):
        head += _s(name) + struct.pack("<I", len(dims))
        for d in dims:
            head += struct.pack("<Q", d)
        head += struct.pack("<IQ", gtype, off)
    pad = (-len(head)) % alignment
    with open(path, "wb") as f:
        f.write(head + b"\0" * pad)
        for _, _, _, data in tensors:
            b = bytes(data)
            f.write(b + b"\0" * ((-len(b)) % alignment))
    return len(head) + pad  # start of the tensor data


def moe_block_tensors(L, block, bias=True, norm=True, router_bias=True, norm_name="post_attention_norm.weight",
                      f16_weights=None, raw_weights=None):
    """Tensors of one transformer block's MoE part from synth.LayerInputs, stacked over
    experts the way the reference's provider slices them (moe_weight_provider.cpp:97-188).
    f16_weights: per expert (w_up [F,H], w_gate [F,H], w_down [H,F]) float16 arrays, written
    as F16 tensors instead of the MXFP4 blocks.  raw_weights: per matrix kind a pair
    (ggml_type, [bytes of expert 0, bytes of expert 1, ...]) written as they are."""
    p = f"blk.{block}"
    t = [(p + ".ffn_gate_inp.weight", GGML_F32, [L.H, L.E], np.ascontiguousarray(L.gate_w, np.float32).tobytes())]
    if router_bias:
        t.append((p + ".ffn_gate_inp.bias", GGML_F32, [L.E], np.ascontiguousarray(L.gate_b, np.float32).tobytes()))
    names = ["ffn_up_exps", "ffn_gate_exps", "ffn_down_exps"]
    for which, nm in enumerate(names):
        rows, K = (L.F, L.H) if which < 2 else (L.H, L.F)
        if raw_weights is not None:
            ty, per_expert = raw_weights[which]
            t.append((f"{p}.{nm}.weight", ty, [K, rows, L.E], b"".join(bytes(x) for x in per_expert)))
        elif f16_weights is not None:
            data = b"".join(np.ascontiguousarray(f16_weights[e][which], np.float16).tobytes() for e in range(L.E))
            t.append((f"{p}.{nm}.weight", GGML_F16, [K, rows, L.E], data))
        else:
            data = b"".join(L.blocks(e, which).tobytes() for e in range(L.E))
            t.append((f"{p}.{nm}.weight", GGML_MXFP4, [K, rows, L.E], data))
        if bias:
            b = (L.b_up, L.b_gate, L.b_down)[which]
            t.append((f"{p}.{nm}.bias", GGML_F32, [rows, L.E], np.ascontiguousarray(b, np.float32).tobytes()))
    if norm:
        t.append((f"{p}.{norm_name}", GGML_F32, [L.H], np.ascontiguousarray(L.norm_w, np.float32).tobytes()))
    return t
