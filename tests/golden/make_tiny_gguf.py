"""Writes a small GGUF v3 file holding the tensors of MoE layers (expert gate / up / down, router, norm, optional shared
expert) by the published container layout: "GGUF", version, counts, key/value entries, tensor infos, zero padding to
general.alignment, tensor data. Independent of the reader under test: plain struct packing. Used by the GGUF tests; run
as a script it writes tests/golden/tiny_moe.gguf (not committed: the tests write their own copy into a temporary folder)."""
import os
import struct
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

GGML_F32, GGML_Q5_1, GGML_Q8_0, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K = 0, 7, 8, 12, 13, 14
BLOCK = {GGML_F32: (1, 4), GGML_Q5_1: (32, 24), GGML_Q8_0: (32, 34), GGML_Q4_K: (256, 144), GGML_Q5_K: (256, 176), GGML_Q6_K: (256, 210)}
U32, F32, STRING, ARRAY, U64, BOOL = 4, 6, 8, 9, 10, 7


def gstr(s):
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def kv(key, vtype, value):
    out = gstr(key) + struct.pack("<I", vtype)
    if vtype == U32:
        return out + struct.pack("<I", value)
    if vtype == U64:
        return out + struct.pack("<Q", value)
    if vtype == F32:
        return out + struct.pack("<f", value)
    if vtype == BOOL:
        return out + struct.pack("<B", value)
    if vtype == STRING:
        return out + gstr(value)
    if vtype == ARRAY:                       # (element type, values): numeric or string elements
        etype, values = value
        body = b"".join(gstr(v) if etype == STRING else struct.pack("<I" if etype == U32 else "<f", v) for v in values)
        return out + struct.pack("<IQ", etype, len(values)) + body
    raise ValueError(vtype)


def write_gguf(path, metadata, tensors, alignment=32, version=3, pad_byte=0, offsets=None):
    """metadata: list of (key, type, value); tensors: list of (name, dims fastest first, ggml type, bytes-like).
    offsets: optional explicit relative offsets (to build invalid files)."""
    head = b"GGUF" + struct.pack("<IQQ", version, len(tensors), len(metadata))
    body = b"".join(kv(*m) for m in metadata)
    infos, rel, at = b"", [], 0
    for n, (name, dims, gtype, data) in enumerate(tensors):
        off = offsets[n] if offsets is not None else at
        rel.append(off)
        infos += gstr(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims) + struct.pack("<IQ", gtype, off)
        at = off + (len(data) + alignment - 1) // alignment * alignment
    blob = head + body + infos
    blob += bytes([pad_byte]) * ((alignment - len(blob) % alignment) % alignment)
    data_offset = len(blob)
    end = max([r + len(t[3]) for r, t in zip(rel, tensors)] + [0])
    section = bytearray(end + (alignment - end % alignment) % alignment)
    for r, t in zip(rel, tensors):
        section[r: r + len(t[3])] = bytes(t[3])
    with open(path, "wb") as f:
        f.write(blob + bytes(section))
    return data_offset, rel


def moe_layer_tensors(rng, layer, hidden, ffn, experts, gate_type=GGML_Q4_K, down_type=GGML_Q4_K, shared_ffn=0, norm=True):
    """Random tensors of one MoE layer: {name: (dims, type, numpy uint8 bytes)} plus the arrays as the tests use them."""
    import orc
    q = {GGML_Q4_K: lambda r, w: orc.quantize_rows(orc.Q4_K, (rng.standard_normal((*r, w)) * 0.05).astype(np.float32)),
         GGML_Q8_0: lambda r, w: orc.quantize_rows(orc.Q8_0, (rng.standard_normal((*r, w)) * 0.05).astype(np.float32)),
         GGML_Q5_K: lambda r, w: orc.random_q5_k(rng, r, w), GGML_Q6_K: lambda r, w: orc.random_q6_k(rng, r, w),
         GGML_Q5_1: lambda r, w: orc.random_q5_1(rng, r, w)}
    p = "blk.%d." % layer
    arrays = {"gate": q[gate_type]((experts, ffn), hidden), "up": q[gate_type]((experts, ffn), hidden), "down": q[down_type]((experts, hidden), ffn),
              "router": (rng.standard_normal((experts, hidden)) * 0.02).astype(np.float32)}
    out = [(p + "ffn_gate_exps.weight", [hidden, ffn, experts], gate_type, arrays["gate"].tobytes()),
           (p + "ffn_up_exps.weight", [hidden, ffn, experts], gate_type, arrays["up"].tobytes()),
           (p + "ffn_down_exps.weight", [ffn, hidden, experts], down_type, arrays["down"].tobytes()),
           (p + "ffn_gate_inp.weight", [hidden, experts], GGML_F32, arrays["router"].tobytes())]
    if norm:
        arrays["norm"] = (1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
        out.append((p + "ffn_norm.weight", [hidden], GGML_F32, arrays["norm"].tobytes()))
    if shared_ffn:
        arrays["shared_gate"], arrays["shared_up"] = q[gate_type]((shared_ffn,), hidden), q[gate_type]((shared_ffn,), hidden)
        arrays["shared_down"] = q[down_type]((hidden,), shared_ffn)
        out += [(p + "ffn_gate_shexp.weight", [hidden, shared_ffn], gate_type, arrays["shared_gate"].tobytes()),
                (p + "ffn_up_shexp.weight", [hidden, shared_ffn], gate_type, arrays["shared_up"].tobytes()),
                (p + "ffn_down_shexp.weight", [shared_ffn, hidden], down_type, arrays["shared_down"].tobytes())]
    return out, arrays


def tiny_moe_file(path, seed=1, hidden=512, ffn=256, experts=6, layers=2, **options):
    rng = np.random.default_rng(seed)
    metadata = [("general.architecture", STRING, "qwen3moe"), ("general.alignment", U32, 64), ("qwen3moe.block_count", U32, layers),
                ("qwen3moe.embedding_length", U32, hidden), ("qwen3moe.expert_feed_forward_length", U32, ffn), ("qwen3moe.expert_count", U32, experts),
                ("qwen3moe.expert_used_count", U32, 2), ("qwen3moe.attention.layer_norm_rms_epsilon", F32, 1e-6),
                ("general.file_type", U64, 15), ("tokenizer.ggml.add_bos_token", BOOL, 1),
                ("tokenizer.ggml.tokens", ARRAY, (STRING, ["a", "bc", "def"])), ("tokenizer.ggml.scores", ARRAY, (F32, [0.5, -1.0, 2.0]))]
    tensors, arrays = [], []
    for layer in range(layers):
        t, a = moe_layer_tensors(rng, layer, hidden, ffn, experts, **options)
        tensors += t
        arrays.append(a)
    data_offset, rel = write_gguf(path, metadata, tensors, alignment=64)
    return metadata, tensors, arrays, data_offset, rel


if __name__ == "__main__":
    here = os.path.dirname(os.path.abspath(__file__))
    tiny_moe_file(os.path.join(here, "tiny_moe.gguf"))
    print("wrote", os.path.join(here, "tiny_moe.gguf"))
