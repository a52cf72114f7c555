"""Writes tests/golden/ref_vectors.npz: outputs of the COMPILED REFERENCE (oracle/_ref/libstrix_ref.so, built from the
reference's own C++ sources by oracle/Makefile) on seeded inputs, so that the oracle can be checked against
reference-produced bits where the reference tree is absent (the GPU box). Inputs are regenerated from the seed by
`cases()`; only expected outputs are stored. Run from the repo root: python tests/golden/make_ref_vectors.py"""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import orc  # noqa: E402


def random_q4k(rng, rows, width):
    """Full-entropy Q4_K bytes with bounded finite fp16 d / dmin (exponent field 3..4, as the reference's device tests use)."""
    w = rng.integers(0, 256, (rows, width // 256 * 144), dtype=np.uint8)
    w[:, 1::144] = (w[:, 1::144] & 0x03) | 0x0C | ((rng.integers(0, 2, w[:, 1::144].shape, dtype=np.uint8)) << 4)
    w[:, 3::144] = (w[:, 3::144] & 0x03) | 0x0C
    return w


def random_q8_0(rng, rows, width):
    w = rng.integers(0, 256, (rows, width // 32 * 34), dtype=np.uint8)
    w[:, 1::34] = (w[:, 1::34] & 0x83) | 0x18
    return w


def layer_case(seed, H, I, E, T, K):
    rng = np.random.default_rng(seed)
    gate = random_q4k(rng, E * I, H).reshape(E, I, -1)
    up = random_q4k(rng, E * I, H).reshape(E, I, -1)
    down = random_q8_0(rng, E * H, I).reshape(E, H, -1)
    x = rng.standard_normal((T, H)).astype(np.float16).astype(np.float32)
    ids = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.uint32)
    return gate, up, down, x, ids


def format_layer_case(seed, H, I, E, T, K):
    """The host executor's other formats: Q5_K gate/up and Q5_1 down blocks of random bytes."""
    rng = np.random.default_rng(seed)
    gate, up = orc.random_q5_k(rng, (E, I), H), orc.random_q5_k(rng, (E, I), H)
    down = orc.random_q5_1(rng, (E, H), I)
    x = rng.standard_normal((T, H)).astype(np.float16).astype(np.float32)
    ids = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.uint32)
    return gate, up, down, x, ids


LAYER_CASES = [(101, 2048, 768, 3, 2, 2), (102, 2560, 640, 2, 3, 2), (103, 512, 256, 6, 4, 3)]
FORMAT_LAYER_CASES = [(111, 1024, 512, 4, 3, 2), (112, 2048, 768, 3, 2, 2)]
Q6K_WIDTHS = [256, 768, 1280, 1536]
RMSNORM_CASES = [(401, 64, 3), (402, 511, 2), (403, 2048, 4), (404, 6144, 2)]
ROW_WIDTHS = [2048, 768, 4096, 5120, 6144, 1280, 27648]
GEMV_CASES = [(201, 4096, 64, 2), (202, 1024, 33, 3)]
# (seed, rows, top_k, width, weights bound, base bound, operands already bfloat16 values): the reference's own two shapes
# (tests/hip_hy4_routed_tests.hip:205-206) and a ragged one with full fp32 operands
COMBINE_CASES = [(501, 5, 16, 1536, True, False, True), (502, 5, 1, 3072, False, True, True), (503, 3, 7, 100, True, True, False),
                 (504, 2, 3, 33, False, False, False)]


def combine_case(seed, rows, top_k, width, has_w, has_base, bf16_operands):
    rng = np.random.default_rng(seed)
    eo = rng.standard_normal((rows, top_k, width)).astype(np.float32)
    base = rng.standard_normal((rows, width)).astype(np.float32)
    if bf16_operands:
        eo = ((eo.view(np.uint32) + 0x8000) & 0xffff0000).astype(np.uint32).view(np.float32)
        base = ((base.view(np.uint32) + 0x8000) & 0xffff0000).astype(np.uint32).view(np.float32)
    w = rng.random((rows, top_k)).astype(np.float32)
    eo[0, 0, 0] = np.float32(np.nan); eo[rows - 1, top_k - 1, width - 1] = np.float32(np.inf)
    eo[0, 0, 1] = np.float32(1.00390625)          # an exact tie of the rounding (1 + 2^-8): to even = 1.0
    eo[0, 0, 2] = np.float32(1.01171875)          # 1 + 3 * 2^-8: to even = 1 + 2^-6
    return eo, (w if has_w else None), (base if has_base else None)


def main():
    R = orc.ref()
    assert R is not None, "build oracle/_ref first (make -C oracle)"
    out = {}
    for seed, H, I, E, T, K in LAYER_CASES:
        gate, up, down, x, ids = layer_case(seed, H, I, E, T, K)
        codes, deltas, sums, _ = orc.quantize_a8(x)
        asg = np.array([[t, k, ids[t, k]] for t in range(T) for k in range(K)], np.uint32)
        raw = np.zeros((T, K, H), np.float32)
        status = np.zeros(T, np.uint32)
        rc = R.ref_routed_expert_run(H, I, gate.ctypes.data_as(orc.u8p), up.ctypes.data_as(orc.u8p), down.ctypes.data_as(orc.u8p),
                                     codes.ctypes.data_as(orc.i8p), deltas.ctypes.data_as(orc.f32p), sums.ctypes.data_as(orc.i32p), T,
                                     asg.ctypes.data_as(orc.u32p), T * K, raw.ctypes.data_as(orc.f32p), C.c_uint64(K * H),
                                     status.ctypes.data_as(orc.u32p), 0, 0)
        assert rc == 0
        out[f"layer_{seed}_rawdots_bits"] = raw.view(np.uint32)
    rng = np.random.default_rng(300)
    vals = []
    o = C.c_float(0)
    for width in ROW_WIDTHS:
        w = random_q4k(rng, 1, width)[0]
        x = rng.standard_normal(width).astype(np.float32)
        codes, deltas, sums, _ = orc.quantize_a8(x[None, :])
        R.ref_gate_row_q4k(w.ctypes.data_as(orc.u8p), width // 256, codes[0].ctypes.data_as(orc.i8p), deltas[0].ctypes.data_as(orc.f32p),
                           sums[0].ctypes.data_as(orc.i32p), C.byref(o))
        vals.append(o.value)
    out["q4k_rows_bits"] = np.array(vals, np.float32).view(np.uint32)
    for seed, width, count, rows in GEMV_CASES:
        rng = np.random.default_rng(seed)
        w = random_q8_0(rng, count, width)
        x = rng.standard_normal((rows, width)).astype(np.float32)
        codes, deltas, sums, _ = orc.quantize_a8(x)
        y = np.zeros((rows, count), np.float32)
        v = orc.Q8a8View(w.ctypes.data, codes.ctypes.data, deltas.ctypes.data, y.ctypes.data, width // 32 * 34, width, count, rows, width, count, 0)
        assert R.ref_gemv_q8_0_a8(C.byref(v)) == 0
        out[f"gemv_{seed}_bits"] = y.view(np.uint32)
        out[f"gemv_{seed}_a8_codes_crc"] = np.array([int(np.bitwise_xor.reduce(codes.view(np.uint8).astype(np.uint32) * np.arange(1, codes.size + 1, dtype=np.uint32).reshape(codes.shape), axis=None))], np.uint32)
    for seed, H, I, E, T, K in FORMAT_LAYER_CASES:
        gate, up, down, x, ids = format_layer_case(seed, H, I, E, T, K)
        codes, deltas, sums, _ = orc.quantize_a8(x)
        asg = np.array([[t, k, ids[t, k]] for t in range(T) for k in range(K)], np.uint32)
        raw = np.zeros((T, K, H), np.float32)
        status = np.zeros(T, np.uint32)
        rc = R.ref_routed_expert_run_fmt(H, I, gate.ctypes.data_as(orc.u8p), up.ctypes.data_as(orc.u8p), down.ctypes.data_as(orc.u8p), 3,
                                         codes.ctypes.data_as(orc.i8p), deltas.ctypes.data_as(orc.f32p), sums.ctypes.data_as(orc.i32p), T,
                                         asg.ctypes.data_as(orc.u32p), T * K, raw.ctypes.data_as(orc.f32p), C.c_uint64(K * H),
                                         status.ctypes.data_as(orc.u32p), 0, 0)
        assert rc == 0
        out[f"format_layer_{seed}_rawdots_bits"] = raw.view(np.uint32)
    rng = np.random.default_rng(310)
    vals = []
    for width in Q6K_WIDTHS:
        w = orc.random_q6_k(rng, (1,), width)[0]
        x = (rng.standard_normal((1, width)) * 3.0).astype(np.float32)
        codes, deltas, sums, _ = orc.quantize_a8(x, tiny_rule=True)
        assert R.ref_evaluate_down_row(w.ctypes.data_as(orc.u8p), C.c_size_t(w.size), codes[0].ctypes.data_as(orc.i8p), deltas[0].ctypes.data_as(orc.f32p),
                                       sums[0].ctypes.data_as(orc.i32p), C.c_size_t(width), 14, C.byref(o)) == 0
        vals.append(o.value)
    out["q6k_down_rows_bits"] = np.array(vals, np.float32).view(np.uint32)
    for seed, n, rows in RMSNORM_CASES:
        rng = np.random.default_rng(seed)
        x = (rng.standard_normal((rows, n)) * 2.0).astype(np.float32)
        w = rng.standard_normal(n).astype(np.float32)
        y = np.empty_like(x)
        assert R.ref_rmsnorm_f32(x.ctypes.data_as(orc.f32p), w.ctypes.data_as(orc.f32p), n, C.c_float(1e-6), y.ctypes.data_as(orc.f32p), rows) == 0
        out[f"rmsnorm_{seed}_bits"] = y.view(np.uint32)
    for case in COMBINE_CASES:
        eo, w, base = combine_case(*case)
        rows, top_k, width = eo.shape
        y = np.zeros((rows, width), np.float32)
        ptr = lambda a: None if a is None else a.ctypes.data_as(orc.f32p)
        assert R.ref_combine_bf16_steps(rows, top_k, width, ptr(w), ptr(eo), ptr(base), ptr(y)) == 0
        out[f"combine_{case[0]}_bits"] = y.view(np.uint32).copy()
        # operands rounded on read == the same combine over operands rounded beforehand (src/moe_core/route_wave_kernel.hpp:96-97)
        R.ref_combine_round_bf16.restype = C.c_float
        rounded = np.array([R.ref_combine_round_bf16(C.c_float(float(v))) if np.isfinite(v) else v for v in eo.ravel()], np.float32).reshape(eo.shape)
        assert R.ref_combine_bf16_steps(rows, top_k, width, ptr(w), ptr(rounded), ptr(base), ptr(y)) == 0
        out[f"combine_{case[0]}_rounded_bits"] = y.view(np.uint32).copy()
    np.savez_compressed(os.path.join(HERE, "ref_vectors.npz"), **out)
    print("wrote", {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
