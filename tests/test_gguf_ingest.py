"""GGUF ingest: header / metadata / tensor-table parsing (CPU) and resident layers
built from a file (GPU).  Files are written by coalsack_amd/gguf_writer.py."""
import numpy as np
import pytest

from coalsack_amd import capi, synth
from coalsack_amd import gguf_writer as gw
from tests.helpers import build_layer, nbits_differ, oracle_layer, assert_layer_close


def _meta(arch="gpt-oss", E=6, k=2, alignment=None):
    m = [("general.architecture", gw.STR, arch),
         ("general.name", gw.STR, "synthetic"),
         (arch + ".expert_count", gw.U32, E),
         (arch + ".expert_used_count", gw.U32, k),
         (arch + ".block_count", gw.U64, 2),
         ("some.i8", gw.I8, -3), ("some.f64", gw.F64, 2.5), ("some.bool", gw.BOOL, 1),
         ("tokenizer.ggml.tokens", gw.ARR, (gw.STR, ["a", "bc", "", "def"])),
         ("tokenizer.ggml.scores", gw.ARR, (gw.F32, [0.5, -1.0, 2.0])),
         ("tokenizer.ggml.token_type", gw.ARR, (gw.I32, [1, 2, 3, 4, 5])),
         ("odd.u16s", gw.ARR, (gw.U16, [7, 8, 9]))]
    if alignment:
        m.append(("general.alignment", gw.U32, alignment))
    return m


@pytest.mark.parametrize("alignment", [None, 64])
def test_parse_header_metadata_and_tensor_table(tmp_path, alignment):
    lib = capi.Library()  # no csk_init: parsing needs no GPU
    L = synth.LayerInputs(6, 2, 64, 96, seed=5, with_norm=True)
    tensors = [("token_embd.weight", gw.GGML_F16, [64, 10], np.zeros(640, np.float16).tobytes())]
    tensors += gw.moe_block_tensors(L, 0) + gw.moe_block_tensors(L, 1, bias=False)
    path = str(tmp_path / "m.gguf")
    data_start = gw.write_gguf(path, _meta(alignment=alignment), tensors, alignment or 32)
    with lib.gguf(path) as g:
        assert g.get_str("general.architecture") == "gpt-oss"
        assert g.get_u32("gpt-oss.expert_count") == 6 and g.get_u32("gpt-oss.block_count") == 2
        assert g.tensor_names() == [t[0] for t in tensors]
        pos = 0
        raw = open(path, "rb").read()
        for name, gtype, dims, data in tensors:
            info = g.tensor_info(name)
            assert info["type"] == gtype and info["dims"] == dims
            assert info["offset"] == data_start + pos and info["nbytes"] == len(data)
            assert raw[info["offset"]:info["offset"] + len(data)] == bytes(data)
            pos += (len(data) + (alignment or 32) - 1) // (alignment or 32) * (alignment or 32)
        up = g.tensor_info("blk.0.ffn_up_exps.weight")
        assert up["nbytes"] == 6 * 96 * (64 // 32) * 17  # experts x rows x blocks x 17 B
        with pytest.raises(capi.CskError, match="Tensor not found"):
            g.tensor_info("blk.9.ffn_up_exps.weight")
        with pytest.raises(capi.CskError, match="Missing required parameter"):
            g.get_u32("gpt-oss.nope")


def test_rejects_bad_files(tmp_path):
    lib = capi.Library()
    p = tmp_path / "bad.gguf"
    p.write_bytes(b"GGML" + b"\0" * 64)
    with pytest.raises(capi.CskError, match="bad magic"):
        lib.gguf(str(p))
    L = synth.LayerInputs(2, 1, 32, 32, seed=1)
    path = str(tmp_path / "t.gguf")
    gw.write_gguf(path, _meta(E=2, k=1), gw.moe_block_tensors(L, 0, norm=False))
    whole = open(path, "rb").read()
    (tmp_path / "cut.gguf").write_bytes(whole[:len(whole) - 40])
    with pytest.raises(capi.CskError, match="past the end"):
        lib.gguf(str(tmp_path / "cut.gguf"))
    (tmp_path / "cut2.gguf").write_bytes(whole[:50])
    with pytest.raises(capi.CskError, match="truncated"):
        lib.gguf(str(tmp_path / "cut2.gguf"))
    with pytest.raises(capi.CskError, match="cannot open"):
        lib.gguf(str(tmp_path / "missing.gguf"))


def test_mutated_files_open_or_are_rejected(tmp_path):
    """Random damage to the header, the key/value section and the tensor table (bytes,
    32- and 64-bit fields set to extreme values, truncation): the parser either reads the
    file or refuses it with a message; it never reads past the file (an AddressSanitizer
    build of the parser ran 24 000 such files clean)."""
    import random
    import struct
    lib = capi.Library()
    L = synth.LayerInputs(2, 1, 32, 32, seed=1)
    path = str(tmp_path / "t.gguf")
    data_start = gw.write_gguf(path, _meta(E=2, k=1), gw.moe_block_tensors(L, 0, norm=False))
    whole = open(path, "rb").read()
    rng = random.Random(7)
    opened = rejected = 0
    for it in range(300):
        b = bytearray(whole)
        mode = it % 4
        if mode == 0:
            for _ in range(rng.randrange(1, 4)):
                b[rng.randrange(data_start)] = rng.randrange(256)
        elif mode == 1:
            pos = rng.randrange(data_start - 8)
            b[pos:pos + 8] = struct.pack("<Q", rng.choice([0, 1, 2**31, 2**32 - 1, 2**40, 2**63, 2**64 - 1]))
        elif mode == 2:
            b = b[:rng.randrange(len(b))]
        else:
            pos = rng.randrange(data_start - 4)
            b[pos:pos + 4] = struct.pack("<I", rng.choice([0, 1, 13, 0xFFFFFFFF, 0x7FFFFFFF]))
        m = tmp_path / "m.gguf"
        m.write_bytes(bytes(b))
        try:
            with lib.gguf(str(m)) as g:
                for name in g.tensor_names():
                    try:
                        g.tensor_info(name)
                    except capi.CskError:
                        pass
            opened += 1
        except capi.CskError as e:
            assert str(e)
            rejected += 1
    assert opened + rejected == 300 and rejected > 100


@pytest.mark.gpu
@pytest.mark.parametrize("T", [5, 90])
def test_layer_from_gguf_equals_layer_built_by_hand(lib, oracle, tmp_path, T):
    """Same bytes through the file and through csk_layer_set_*: identical resident
    weights and bit-identical outputs; and the file-built layer matches the CPU path."""
    E, k, H, F = 6, 2, 96, 160
    L0 = synth.LayerInputs(E, k, H, F, seed=11, with_norm=True)
    L1 = synth.LayerInputs(E, k, H, F, seed=12, layer=1, with_norm=True)
    path = str(tmp_path / "two_blocks.gguf")
    gw.write_gguf(path, _meta(E=E, k=k), gw.moe_block_tensors(L0, 0) + gw.moe_block_tensors(L1, 1, bias=False))
    hidden = synth.hidden_states(T, H, seed=3)
    flags = capi.FWD_RMSNORM | capi.FWD_RESIDUAL
    with lib.gguf(path) as g:
        for blk, L, bias in ((0, L0, True), (1, L1, False)):
            with g.layer(blk) as layer, build_layer(lib, L, bias=bias, norm=True) as hand:
                assert (layer.E, layer.k, layer.H, layer.F) == (E, k, H, F)
                for e in (0, E - 1):
                    for which in range(3):
                        assert np.array_equal(layer.export(e, which), L.blocks(e, which))
                got = layer.forward(hidden, flags)
                assert nbits_differ(got, hand.forward(hidden, flags)) == 0
                want, _ = oracle_layer(oracle, L, hidden, bias=bias, norm=True, residual=True)
                assert_layer_close(got, want)


@pytest.mark.gpu
def test_layer_from_gguf_llama4_switches_and_errors(lib, oracle, tmp_path):
    E, k, H, F = 4, 1, 64, 64
    L = synth.LayerInputs(E, k, H, F, seed=21, with_norm=True)
    path = str(tmp_path / "l4.gguf")
    gw.write_gguf(path, _meta("llama4", E, k),
                  gw.moe_block_tensors(L, 0, bias=False, router_bias=False, norm_name="ffn_norm.weight"))
    hidden = synth.hidden_states(7, H, seed=4)
    with lib.gguf(path) as g, g.layer(0) as layer:
        got = layer.forward(hidden, capi.FWD_RMSNORM)
    L.gate_b = np.zeros(E, np.float32)
    # llama4: sigmoid gating, weight before the FFN, standard SwiGLU (llm_engine.cpp:145-161, 738-740)
    want, _ = oracle_layer(oracle, L, hidden, bias=False, norm=True, sigmoid=True, weight_before_ffn=True,
                           act=1)
    assert_layer_close(got, want)
    # expert tensors of mixed or unsupported types are refused, not misread
    mixed = gw.moe_block_tensors(L, 0, bias=False, router_bias=False)
    mixed[1] = (mixed[1][0], gw.GGML_F16, mixed[1][2], np.zeros(E * F * H, np.float16).tobytes())
    gw.write_gguf(str(tmp_path / "mixed.gguf"), _meta(E=E, k=k), mixed)
    # Q5_K (type 13): 176 bytes per 256 elements
    q4 = [(n, 13, d, bytes(int(np.prod(d)) // 256 * 176)) if "_exps.weight" in n else (n, t, d, b)
          for n, t, d, b in gw.moe_block_tensors(L, 0, bias=False, router_bias=False)]
    gw.write_gguf(str(tmp_path / "q4k.gguf"), _meta(E=E, k=k), q4)
    with lib.gguf(str(tmp_path / "mixed.gguf")) as g:
        with pytest.raises(capi.CskError, match="must be all MXFP4"):
            g.layer(0)
        with pytest.raises(capi.CskError, match="Tensor not found"):
            g.layer(3)
    with lib.gguf(str(tmp_path / "q4k.gguf")) as g:
        with pytest.raises(capi.CskError, match="only MXFP4, F16, Q4_K and Q6_K"):
            g.layer(0)


@pytest.mark.gpu
@pytest.mark.parametrize("T", [5, 90])
def test_layer_from_gguf_f16_experts(lib, oracle, tmp_path, T):
    """A block whose expert tensors are F16: the file-built layer holds the file's halves,
    equals a layer built through csk_layer_set_expert_f16 bit for bit, and matches the CPU
    path's float16 branch."""
    from tests.test_oracle_expert_f16 import random_f16_expert
    E, k, H, F = 6, 2, 96, 160
    L = synth.LayerInputs(E, k, H, F, seed=41, with_norm=True)
    rng = np.random.default_rng(41)
    ws = [random_f16_expert(rng, H, F, 0.1) for _ in range(E)]
    path = str(tmp_path / "f16.gguf")
    gw.write_gguf(path, _meta(E=E, k=k), gw.moe_block_tensors(L, 0, f16_weights=ws))
    hidden = synth.hidden_states(T, H, seed=5)
    flags = capi.FWD_RMSNORM | capi.FWD_RESIDUAL
    with lib.gguf(path) as g:
        with g.layer(0) as layer, lib.layer(E, k, H, F, f16=True) as hand:
            assert layer.f16 and (layer.E, layer.k, layer.H, layer.F) == (E, k, H, F)
            hand.set_router(L.gate_w, L.gate_b)
            hand.set_norm(L.norm_w, 1e-5)
            for e in range(E):
                hand.set_expert_f16(e, *ws[e], L.b_up[e], L.b_gate[e], L.b_down[e])
                for which in range(3):
                    assert np.array_equal(layer.export_f16(e, which).view(np.uint16),
                                          ws[e][which].view(np.uint16))
            got = layer.forward(hidden, flags)
            assert nbits_differ(got, hand.forward(hidden, flags)) == 0
    want, _ = oracle.moe_layer(hidden, E, k, H, F, L.gate_w, L.gate_b, np.stack([w[0] for w in ws]),
                               np.stack([w[1] for w in ws]), np.stack([w[2] for w in ws]), L.b_up,
                               L.b_gate, L.b_down, norm_w=L.norm_w, norm_eps=1e-5, residual=True)
    assert_layer_close(got, want)


@pytest.mark.gpu
def test_layer_from_gguf_kquant_experts(lib, oracle, tmp_path):
    """A block in the style of a Q4_K_M checkpoint: gate and up experts Q4_K, down experts
    Q6_K.  The resident halves equal what the reference's weight provider hands to the node
    (K-quant -> fp32 -> truncating fp16), and the forward matches the CPU path's float16
    branch over those halves."""
    from tests.golden.make_kquant_golden import random_blocks
    E, k, H, F = 4, 2, 128, 256
    L = synth.LayerInputs(E, k, H, F, seed=51, with_norm=True)
    rng = np.random.default_rng(51)
    nsb = H * F // 256
    raw = [(12, [random_blocks(rng, "q4_k", nsb).tobytes() for _ in range(E)]),
           (12, [random_blocks(rng, "q4_k", nsb).tobytes() for _ in range(E)]),
           (14, [random_blocks(rng, "q6_k", nsb).tobytes() for _ in range(E)])]
    path = str(tmp_path / "q4km.gguf")
    gw.write_gguf(path, _meta(E=E, k=k), gw.moe_block_tensors(L, 0, raw_weights=raw))
    halves = [[oracle.kquant_to_fp16("q4_k" if raw[w][0] == 12 else "q6_k",
                                     np.frombuffer(raw[w][1][e], np.uint8), H * F)
               .reshape((H, F) if w == 2 else (F, H)) for w in range(3)] for e in range(E)]
    hidden = synth.hidden_states(9, H, seed=6)
    with lib.gguf(path) as g, g.layer(0) as layer:
        assert layer.f16
        for e in range(E):
            for w in range(3):
                assert np.array_equal(layer.export_f16(e, w).view(np.uint16), halves[e][w])
        got = layer.forward(hidden, capi.FWD_RMSNORM)
    stack = lambda w: np.stack([halves[e][w] for e in range(E)]).view(np.float16)
    want, _ = oracle.moe_layer(hidden, E, k, H, F, L.gate_w, L.gate_b, stack(0), stack(1), stack(2), L.b_up,
                               L.b_gate, L.b_down, norm_w=L.norm_w, norm_eps=1e-5)
    assert np.all(np.isfinite(want))
    assert_layer_close(got, want)


@pytest.mark.gpu
def test_layer_from_split_checkpoint_equals_single_file(lib, tmp_path):
    """A block whose tensors are spread over two shard files (gguf_multi_loader,
    moe_weight_provider.cpp:75-100): every tensor is read from its own shard, and the layer is
    bit-identical to the one built from a single file."""
    E, k, H, F = 6, 2, 96, 160
    L = synth.LayerInputs(E, k, H, F, seed=31, with_norm=True)
    tensors = gw.moe_block_tensors(L, 0)
    one = str(tmp_path / "one.gguf")
    gw.write_gguf(one, _meta(E=E, k=k), tensors)
    first = [t for t in tensors if "ffn_up" in t[0] or "gate_inp" in t[0]]
    second = [t for t in tensors if t not in first]
    a, b = str(tmp_path / "s-00001-of-00002.gguf"), str(tmp_path / "s-00002-of-00002.gguf")
    gw.write_gguf(a, _meta(E=E, k=k), [("pad.weight", gw.GGML_F32, [7], np.zeros(7, np.float32).tobytes())] + first)
    gw.write_gguf(b, [("general.architecture", gw.STR, "gpt-oss")], second)
    hidden = synth.hidden_states(9, H, seed=5)
    flags = capi.FWD_RMSNORM | capi.FWD_RESIDUAL
    with lib.gguf(one) as g1, lib.gguf([a, b]) as g2:
        assert g2.tensor_shard("blk.0.ffn_down_exps.weight") == 1 and g2.tensor_shard("blk.0.ffn_up_exps.weight") == 0
        with g1.layer(0) as l1, g2.layer(0) as l2:
            for e in (0, E - 1):
                for which in range(3):
                    assert np.array_equal(l2.export(e, which), L.blocks(e, which))
            assert nbits_differ(l2.forward(hidden, flags), l1.forward(hidden, flags)) == 0
