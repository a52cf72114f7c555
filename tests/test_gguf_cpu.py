"""The GGUF v3 reader and the MoE layer map: the byte fixtures the reference's own reader tests build (tests/core_tests.cpp:56-126
with the outcomes of :289-370, tests/gguf_pack_writer_test.cpp:19-31), files written by tests/golden/make_tiny_gguf.py (an
independent writer following the published container layout), and the reader's refusals: the rules of the reference reader
(src/gguf_reader.cpp:22-90, 130-260, 296-360). Host code only."""
import os
import struct
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
import make_tiny_gguf as mk


@pytest.fixture(scope="module")
def pkg():
    from __graft_entry__ import load_package
    return load_package()


def test_index_metadata_and_layer_map(pkg, tmp_path):
    path = str(tmp_path / "tiny.gguf")
    metadata, tensors, arrays, data_offset, rel = mk.tiny_moe_file(path, shared_ffn=256)
    g = pkg.GgufFile(path)
    assert g.alignment == 64 and g.data_offset == data_offset and data_offset % 64 == 0
    got = g.tensors()
    assert len(got) == len(tensors)
    for t, (name, dims, gtype, data), r in zip(got, tensors, rel):
        assert t == {"name": name, "dims": dims, "type": gtype, "offset": data_offset + r, "bytes": len(data)}
        assert np.array_equal(g.read(pkg.GgufTensor(name.encode(), len(dims), (pkg.C.c_uint64 * 4)(*dims), gtype, t["offset"], t["bytes"])).numpy(),
                              np.frombuffer(data, np.uint8))
    assert g.metadata("general.architecture") == "qwen3moe" and g.metadata("qwen3moe.expert_count") == 6
    assert g.metadata("general.file_type") == 15 and g.metadata("tokenizer.ggml.add_bos_token") == 1
    assert abs(g.metadata("qwen3moe.attention.layer_norm_rms_epsilon") - 1e-6) < 1e-12
    assert g.metadata("tokenizer.ggml.tokens") == 3 and g.metadata("tokenizer.ggml.scores") == 3        # arrays: their length
    with pytest.raises(pkg.StrixError):
        g.metadata("no.such.key")
    for layer in (0, 1):
        m = g.moe_layer_map(layer)
        assert (m.hidden, m.ffn, m.experts, m.shared_ffn, m.gate_type, m.down_type) == (512, 256, 6, 256, 12, 12)
        assert m.gate.name == b"blk.%d.ffn_gate_exps.weight" % layer and m.gate.bytes == 6 * 256 * 2 * 144
        assert np.array_equal(g.read(m.down).numpy(), arrays[layer]["down"].reshape(-1))
        assert np.array_equal(g.read(m.router).view(pkg.torch.float32).numpy(), arrays[layer]["router"].reshape(-1))
        assert m.norm.bytes == 4 * 512 and m.router_bias.bytes == 0 and m.shared_down.bytes == 512 * 144 and m.shared_router.bytes == 0
    with pytest.raises(pkg.StrixError):
        g.moe_layer_map(2)
    g.close()


def rewrite(path, mutate):
    raw = bytearray(open(path, "rb").read())
    mutate(raw)
    open(path, "wb").write(bytes(raw))


def refused(pkg, path, reason):
    with pytest.raises(pkg.StrixError) as e:
        pkg.GgufFile(path)
    assert reason in str(e.value), str(e.value)


def test_reader_refusals(pkg, tmp_path):
    rng = np.random.default_rng(3)
    path = str(tmp_path / "bad.gguf")
    t32 = lambda name, n: (name, [n], mk.GGML_F32, np.zeros(n, np.float32).tobytes())
    base_meta = [("general.architecture", mk.STRING, "x")]
    ok = [t32("a", 8), t32("b", 16)]
    mk.write_gguf(path, base_meta, ok)
    assert len(pkg.GgufFile(path).tensors()) == 2
    rewrite(path, lambda raw: raw.__setitem__(slice(0, 4), b"GGML"))
    refused(pkg, path, "invalid GGUF magic")
    mk.write_gguf(path, base_meta, ok, version=2)
    refused(pkg, path, "only GGUF v3")
    mk.write_gguf(path, base_meta, ok, pad_byte=1)
    refused(pkg, path, "padding must contain zero")
    mk.write_gguf(path, base_meta, ok, offsets=[0, 8])
    refused(pkg, path, "offset is not aligned")
    mk.write_gguf(path, base_meta, ok, offsets=[0, 0])
    refused(pkg, path, "overlap")
    mk.write_gguf(path, base_meta, [t32("a", 8), t32("a", 8)])
    refused(pkg, path, "duplicate GGUF tensor name")
    mk.write_gguf(path, base_meta + base_meta, ok)
    refused(pkg, path, "duplicate GGUF metadata key")
    mk.write_gguf(path, [("General.Architecture", mk.STRING, "x")], ok)
    refused(pkg, path, "invalid GGUF metadata key")
    mk.write_gguf(path, [("a..b", mk.STRING, "x")], ok)
    refused(pkg, path, "invalid GGUF metadata key")
    mk.write_gguf(path, base_meta + [("general.alignment", mk.U32, 12)], ok, alignment=12)
    refused(pkg, path, "multiple of 8")
    mk.write_gguf(path, base_meta + [("general.alignment", mk.STRING, "32")], ok)
    refused(pkg, path, "must be an unsigned integer")
    mk.write_gguf(path, base_meta + [("some.flag", mk.BOOL, 2)], ok)
    refused(pkg, path, "boolean must be zero or one")
    mk.write_gguf(path, base_meta, [("q", [100], mk.GGML_Q4_K, bytes(144))])
    refused(pkg, path, "not divisible by its quantization block")
    for removed in (4, 5, 31, 36, 40, 99):
        mk.write_gguf(path, base_meta, [("q", [32], removed, bytes(64))])
        refused(pkg, path, "unsupported or removed GGML tensor type")
    mk.write_gguf(path, base_meta, [("z", [8, 0], mk.GGML_F32, bytes(32))])
    refused(pkg, path, "dimensions must be non-zero")
    mk.write_gguf(path, base_meta, [("r", [2, 2, 2, 2, 2], mk.GGML_F32, bytes(128))])
    refused(pkg, path, "dimension count is invalid")
    mk.write_gguf(path, base_meta, ok)
    rewrite(path, lambda raw: raw.__delitem__(slice(len(raw) - 40, len(raw))))          # the last tensor runs past the end
    refused(pkg, path, "exceeds file size")
    mk.write_gguf(path, base_meta, ok)
    rewrite(path, lambda raw: raw.__delitem__(slice(30, len(raw))))                     # cut inside the metadata
    refused(pkg, path, "unexpected end of GGUF file")
    with pytest.raises(pkg.StrixError):
        pkg.GgufFile(str(tmp_path / "missing.gguf"))


def test_layer_map_refusals(pkg, tmp_path):
    rng = np.random.default_rng(4)
    path = str(tmp_path / "layer.gguf")
    tensors, _ = mk.moe_layer_tensors(rng, 0, 256, 256, 2)
    meta = [("general.architecture", mk.STRING, "x")]

    def layer_refused(ts, reason):
        mk.write_gguf(path, meta, ts)
        g = pkg.GgufFile(path)
        with pytest.raises(pkg.StrixError) as e:
            g.moe_layer_map(0)
        assert reason in str(e.value), str(e.value)

    layer_refused([t for t in tensors if "ffn_up_exps" not in t[0]], "not all present")
    swapped = [(n, ([256, 256, 3] if "ffn_up_exps" in n else d), t, (b + b[: len(b) // 2] if "ffn_up_exps" in n else b)) for n, d, t, b in tensors]
    layer_refused(swapped, "same shape and type")
    wrong_router = [(n, ([256, 3] if "gate_inp" in n else d), t, (bytes(256 * 3 * 4) if "gate_inp" in n else b)) for n, d, t, b in tensors]
    layer_refused(wrong_router, "router must be an F32")
    down_f32 = [(n, d, (0 if "down_exps" in n else t), (bytes(256 * 256 * 2 * 4) if "down_exps" in n else b)) for n, d, t, b in tensors]
    layer_refused(down_f32, "down experts must be")


# ---- the reference's own byte fixtures -------------------------------------------------------------------------------
def _le(fmt, v):
    return struct.pack("<" + fmt, v)


def _s(text):
    return _le("Q", len(text)) + text.encode()


def ref_valid_gguf(tensor_offset=0, tensor_type=1):
    """valid_gguf of tests/core_tests.cpp:56-82: two metadata values, one tensor [16, 32] of `tensor_type`, 1024 data bytes."""
    b = b"GGUF" + _le("I", 3) + _le("Q", 1) + _le("Q", 2)
    b += _s("general.architecture") + _le("I", 8) + _s("qwen4exp")
    b += _s("general.alignment") + _le("I", 4) + _le("I", 32)
    b += _s("blk.0.weight") + _le("I", 2) + _le("Q", 16) + _le("Q", 32) + _le("I", tensor_type) + _le("Q", tensor_offset)
    b += bytes(-len(b) % 32)
    return b + bytes(1024)


def ref_array_gguf():
    """array_gguf of tests/core_tests.cpp:84-99: one metadata array of three uint32."""
    b = b"GGUF" + _le("I", 3) + _le("Q", 0) + _le("Q", 1)
    b += _s("test.values") + _le("I", 9) + _le("I", 4) + _le("Q", 3) + _le("I", 10) + _le("I", 20) + _le("I", 30)
    return b + bytes(-len(b) % 32)


def ref_two_tensor_gguf(second_offset):
    """two_tensor_gguf of tests/core_tests.cpp:101-121: two F16 tensors [16, 32] (1024 bytes each), 2048 data bytes."""
    b = b"GGUF" + _le("I", 3) + _le("Q", 2) + _le("Q", 0)
    for name, offset in (("first.weight", 0), ("second.weight", second_offset)):
        b += _s(name) + _le("I", 2) + _le("Q", 16) + _le("Q", 32) + _le("I", 1) + _le("Q", offset)
    b += bytes(-len(b) % 32)
    return b + bytes(2048)


def ref_pack_writer_source():
    """The source file of tests/gguf_pack_writer_test.cpp:19-31: a string and a uint32, an F32 [4] and a BF16 [128, 16] tensor."""
    b = b"GGUF" + _le("I", 3) + _le("Q", 2) + _le("Q", 2)
    b += _s("general.architecture") + _le("I", 8) + _s("qwen35")
    b += _s("qwen35.block_count") + _le("I", 4) + _le("I", 7)
    b += _s("norm.weight") + _le("I", 1) + _le("Q", 4) + _le("I", 0) + _le("Q", 0)
    b += _s("w.weight") + _le("I", 2) + _le("Q", 128) + _le("Q", 16) + _le("I", 30) + _le("Q", 32)
    b += bytes(-len(b) % 32)
    return b + b"n" * 16 + bytes(16) + b"w" * 4096


def test_reference_reader_fixtures(pkg, tmp_path):
    """The reference's parse results and refusals on its own fixtures (tests/core_tests.cpp:289-370). Not replayed: the two cases
    that pass a Limits object (max_string_bytes = 4, max_total_array_elements = 2) - this reader's limits are fixed."""
    path = str(tmp_path / "ref.gguf")

    def opened(raw):
        open(path, "wb").write(raw)
        return pkg.GgufFile(path)

    def refuses(raw, reason):
        open(path, "wb").write(raw)
        refused(pkg, path, reason)

    raw = ref_valid_gguf()
    g = opened(raw)
    assert g.alignment == 32 and len(g.tensors()) == 1                                    # "GGUF alignment metadata is applied", "tensor directory parses"
    assert int(pkg.lib().mi355_gguf_metadata_count(g.handle)) == 2                        # "metadata count is preserved"
    t = g.tensors()[0]
    assert t["offset"] == g.data_offset and g.data_offset % 32 == 0                       # "relative tensor offset resolves from data section"
    assert t["bytes"] == 1024 and t["offset"] + t["bytes"] == len(raw)                    # "F16 tensor range is computed exactly"
    assert t["name"] == "blk.0.weight" and t["dims"] == [16, 32] and t["type"] == 1
    assert g.metadata("general.architecture") == "qwen4exp"                               # "architecture metadata is available"
    g.close()
    refuses(b"B" + raw[1:], "invalid GGUF magic")                                         # "rejects invalid magic"
    refuses(ref_valid_gguf(1), "offset is not aligned")                                   # "rejects unaligned tensor offsets"
    refuses(ref_valid_gguf(0, 31), "unsupported or removed GGML tensor type")             # "rejects removed tensor types"
    refuses(ref_valid_gguf(0, 2), "not divisible by its quantization block")              # "rows not divisible by quantization block size"
    refuses(raw[:-1], "exceeds file size")                                                # "tensor ranges extending beyond the file"
    g = opened(ref_two_tensor_gguf(1024))
    first, second = g.tensors()
    assert second["offset"] == first["offset"] + first["bytes"]                           # "permits adjacent non-overlapping tensor ranges"
    g.close()
    refuses(ref_two_tensor_gguf(0), "overlap")                                            # "rejects overlapping tensor data ranges"
    flag = b"GGUF" + _le("I", 3) + _le("Q", 0) + _le("Q", 1) + _s("test.flag") + _le("I", 7) + _le("B", 2)
    refuses(flag + bytes(-len(flag) % 32), "boolean must be zero or one")                 # "rejects non-canonical booleans"
    g = opened(ref_array_gguf())
    assert g.metadata("test.values") == 3 and len(g.tensors()) == 0                       # "array summary parses without retaining its payload"
    g.close()
    # the pack writer's source file: 32-byte default alignment, an F32 and a BF16 tensor with a gap between them
    raw = ref_pack_writer_source()
    g = opened(raw)
    norm, wt = g.tensors()
    assert g.alignment == 32 and g.metadata("qwen35.block_count") == 7 and g.metadata("general.architecture") == "qwen35"
    assert (norm["name"], norm["dims"], norm["type"], norm["bytes"], norm["offset"]) == ("norm.weight", [4], 0, 16, g.data_offset)
    assert (wt["name"], wt["dims"], wt["type"], wt["bytes"], wt["offset"]) == ("w.weight", [128, 16], 30, 4096, g.data_offset + 32)
    assert wt["offset"] + wt["bytes"] == len(raw)
    assert bytes(g.read(pkg.GgufTensor(b"norm.weight", 1, (pkg.C.c_uint64 * 4)(4), 0, norm["offset"], 16)).numpy()) == b"n" * 16
    g.close()
