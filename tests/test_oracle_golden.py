"""Pins the CPU oracle (oracle/strix_oracle.c) WITHOUT the GPU:
  * the literal vectors the reference's own host tests hold for this path (tests/golden/reference_literals.json),
  * closed forms / brute force / invariants chosen so that a plausible mistake fails,
  * mutation checks (a wrong order, a fused multiply-add, a swapped nibble must change the bits),
  * bitwise equality with the compiled reference (oracle/_ref) where that library was built,
  * the committed reference-generated vectors (tests/golden/ref_vectors.npz)."""
import json
import math
import os

import numpy as np
import pytest

import orc

HERE = os.path.dirname(os.path.abspath(__file__))
LIT = json.load(open(os.path.join(HERE, "golden", "reference_literals.json")))


def f32_from_bits(b):
    return np.array([int(b, 16) if isinstance(b, str) else b], np.uint32).view(np.float32)[0]


def bits(x):
    return np.asarray(x, np.float32).view(np.uint32)


# ---------------------------------------------------------------- fp16
def test_half_to_float_all_65536_values():
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([orc.half_to_float(int(v)) for v in h], np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(bits(got)[~nan], bits(want)[~nan])


def test_float_to_half_round_trip_and_ties():
    h = np.arange(65536, dtype=np.uint16)
    f = h.view(np.float16).astype(np.float32)
    ok = ~np.isnan(f)
    back = np.array([orc.float_to_half(v) for v in f[ok]], np.uint16)
    assert np.array_equal(back, h[ok])
    rng = np.random.default_rng(5)
    sample = np.concatenate([rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32),
                             # exact midpoints between neighbouring halves: ties must go to even
                             ((f[ok][:-1].astype(np.float64) + f[ok][1:].astype(np.float64)) / 2).astype(np.float32)[::7]])
    sample = sample[np.isfinite(sample)]
    with np.errstate(over="ignore"):
        want = sample.astype(np.float16).view(np.uint16)
    got = np.array([orc.float_to_half(v) for v in sample], np.uint16)
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- Q8_0 decode / writer
def test_q8_0_dequant_closed_form():
    rng = np.random.default_rng(1)
    raw = rng.integers(0, 256, (5, 4 * 34), dtype=np.uint8)
    raw[:, 1::34] &= 0x7B  # finite scales
    got = orc.dequant_rows(orc.Q8_0, raw, 128)
    blocks = raw.reshape(5, 4, 34)
    d = blocks[:, :, :2].copy().view(np.float16).astype(np.float32)
    want = (blocks[:, :, 2:].view(np.int8).astype(np.float32) * d).reshape(5, 128)
    assert np.array_equal(bits(got), bits(want))


def test_q8_0_writer_reference_literals():
    for case in LIT["q8_0_writer"]["cases"]:
        v = np.zeros(32, np.float32)
        if case.get("ramp"):
            v = (np.arange(32) - 16).astype(np.float32)
        for k, x in case.get("values", {}).items():
            v[int(k)] = x
        packed = orc.quantize_rows(orc.Q8_0, v[None, :])[0]
        d = np.float32(case["d"]) if "d" in case else np.float32(case["d_num"]) / np.float32(case["d_den"])
        assert packed[:2].view(np.uint16)[0] == orc.float_to_half(d), case["name"]
        codes = packed[2:].view(np.int8)
        for k, c in case["codes"].items():
            assert codes[int(k)] == c, (case["name"], k)


# ---------------------------------------------------------------- Q4_K decode
def _independent_q4k_value(block, k):
    """Element k of one 144-byte block from the published layout, written element-wise (no loops shared with the oracle)."""
    g, l = k // 32, k % 32
    s = block[4:16].astype(np.uint32)
    if g < 4:
        sc, m = s[g] & 63, s[g + 4] & 63
    else:
        sc = (s[g + 4] & 15) | ((s[g - 4] >> 6) << 4)
        m = (s[g + 4] >> 4) | ((s[g] >> 6) << 4)
    d = block[0:2].copy().view(np.float16)[0].astype(np.float32)
    dm = block[2:4].copy().view(np.float16)[0].astype(np.float32)
    q = (int(block[16 + 32 * (g // 2) + l]) >> (4 * (g % 2))) & 15
    return np.float32(np.float32(d * np.float32(sc)) * np.float32(q)) - np.float32(dm * np.float32(m))


def test_q4k_dequant_every_position_brute_force():
    rng = np.random.default_rng(2)
    raw = rng.integers(0, 256, (3, 2 * 144), dtype=np.uint8)
    for r in range(3):
        for b in range(2):
            raw[r, b * 144 + 1] &= 0x7B
            raw[r, b * 144 + 3] &= 0x7B
    got = orc.dequant_rows(orc.Q4_K, raw, 512)
    for r in range(3):
        for k in range(512):
            want = _independent_q4k_value(raw[r, (k // 256) * 144:(k // 256 + 1) * 144], k % 256)
            assert bits(got[r, k]) == bits(want), (r, k)


def test_q4k_factor_unpack_all_scale_min_group_triples():
    """Both statements of the 6-bit unpack (byte form and 32-bit-word form) against every (scale, min, group)
    (the reference sweeps the same 64 x 64 x 8 triples: tests/moe_q4k_a8_contract_tests.cpp:103-118)."""
    import ctypes as C
    L = orc.lib()
    rng = np.random.default_rng(3)
    block = np.zeros(144, np.uint8)
    sc_out, m_out = C.c_uint8(0), C.c_uint8(0)
    for group in range(8):
        lo = group & 3
        for s in range(64):
            for m in range(64):
                p = rng.integers(0, 256, 12, dtype=np.uint8)
                if group < 4:
                    p[lo] = (p[lo] & 192) | s
                    p[lo + 4] = (p[lo + 4] & 192) | m
                else:
                    p[lo] = (p[lo] & 63) | ((s >> 4) << 6)
                    p[lo + 4] = (p[lo + 4] & 63) | ((m >> 4) << 6)
                    p[lo + 8] = (s & 15) | ((m & 15) << 4)
                block[4:16] = p
                L.orc_q4k_scale_min(block[4:].ctypes.data_as(orc.u8p), group, C.byref(sc_out), C.byref(m_out))
                assert (sc_out.value, m_out.value) == (s, m)
                assert L.orc_q4k_factor_words(block.ctypes.data_as(orc.u8p), group, 0) == s
                assert L.orc_q4k_factor_words(block.ctypes.data_as(orc.u8p), group, 1) == m


def test_q4k_writer_round_trip_error_bound():
    """The writer has no reference counterpart (parity unpinned); it must still produce valid blocks whose decode is
    within one quantisation step of the input."""
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((4, 1024)) * 0.02).astype(np.float32)
    x[1, :32] = 0.0
    x[2, 256:512] = np.abs(x[2, 256:512])
    packed = orc.quantize_rows(orc.Q4_K, x)
    y = orc.dequant_rows(orc.Q4_K, packed, 1024)
    span = (x.reshape(4, -1, 32).max(-1) - np.minimum(x.reshape(4, -1, 32).min(-1), 0)).repeat(32, -1).reshape(4, 1024)
    assert np.all(np.abs(x - y) <= span / 15 * 0.75 + 1e-6)


# ---------------------------------------------------------------- A8 quantiser
def test_a8_reference_literals():
    for case in LIT["a8_quantiser"]["cases"]:
        w = case["width"]
        v = np.full(w, f32_from_bits(case["fill_bits"]) if "fill_bits" in case else case["fill"], np.float32)
        for k, x in case.get("set", {}).items():
            v[int(k)] = x
        for k, b in case.get("set_bits", {}).items():
            v[int(k)] = f32_from_bits(b)
        codes, deltas, sums, rc = orc.quantize_a8(v[None, :], tiny_rule=case.get("tiny_rule", False))
        src = case["source"]
        if "all_codes" in case:
            assert np.all(codes == case["all_codes"]), src
        for k, c in case.get("codes", {}).items():
            assert codes[0, int(k)] == c, (src, k)
        if "delta" in case:
            assert np.all(deltas == np.float32(case["delta"])), src
        if "delta_not" in case:
            assert deltas[0, 0] != np.float32(case["delta_not"]), src
        if "delta_bits" in case:
            assert bits(deltas[0, 0]) == int(case["delta_bits"], 16), src
        if "sum" in case:
            assert np.all(sums == case["sum"]), src


def _rne_ratio(n, d):
    q, r = divmod(n, d)
    if r * 2 > d or (r * 2 == d and (q & 1)):
        q += 1
    return q


def _soft_divide(a, b):
    """Correctly rounded binary32 quotient from integer significands (independent of the native divide);
    the reference carries the same construction in tests/q4k_a8_oracle.hpp:20-45."""
    sign = (a ^ b) & 0x80000000
    a &= 0x7FFFFFFF
    b &= 0x7FFFFFFF
    if a == 0:
        return sign

    def unpack(x):
        e = x >> 23
        m = (x & 0x7FFFFF) | (0x800000 if e else 0)
        ex = e - 150 if e else -149
        sh = 24 - m.bit_length()
        return m << sh, ex - sh
    ma, ea = unpack(a)
    mb, eb = unpack(b)
    diff = ea - eb
    exponent = diff + (-1 if ma < mb else 0)
    if exponent < -126:
        shift = diff + 149
        if shift < -1:
            return sign
        return sign | _rne_ratio(ma << max(shift, 0), mb << max(-shift, 0))
    if exponent > 127:
        return sign | 0x7F800000
    m = _rne_ratio(ma << (diff - exponent + 23), mb)
    if m == 0x1000000:
        m >>= 1
        exponent += 1
    if exponent > 127:
        return sign | 0x7F800000
    return sign | ((exponent + 127) << 23) | (m - 0x800000)


def test_a8_against_software_division_at_rounding_boundaries():
    rng = np.random.default_rng(6)
    for _ in range(300):
        amax_bits = int(rng.integers(0x20000000, 0x7F000000))
        dbits = _soft_divide(amax_bits, 0x42FE0000)
        delta = f32_from_bits(dbits)
        amax = f32_from_bits(amax_bits)
        v = np.zeros(32, np.float32)
        v[0] = amax
        for lane in range(1, 32):
            boundary = np.float32(delta * np.float32(lane + 0.5))
            x = np.nextafter(boundary, np.float32(0.0) if lane & 1 else amax)
            v[lane] = -min(amax, x) if lane & 2 else min(amax, x)
        codes, deltas, sums, _ = orc.quantize_a8(v[None, :], tiny_rule=False)
        assert bits(deltas[0, 0]) == dbits
        for lane in range(32):
            qb = _soft_divide(int(bits(v[lane])), dbits)
            mag = abs(float(f32_from_bits(qb)))
            c = math.floor(mag)
            frac = mag - c
            if frac > 0.5 or (frac == 0.5 and (c & 1)):
                c += 1
            c = min(c, 127)
            assert codes[0, lane] == (-c if qb & 0x80000000 else c)
        assert sums[0, 0] == int(codes.astype(np.int32).sum())


def test_a8_rejects_partial_group_before_any_write():
    x = np.ones(64, np.float32)
    import ctypes as C
    codes = np.full(64, 17, np.int8)
    deltas = np.full(2, 19, np.float32)
    sums = np.full(2, 23, np.int32)
    for width in (31, 33):
        rc = orc.lib().orc_quantize_a8(x.ctypes.data_as(orc.f32p), C.c_size_t(width), codes.ctypes.data_as(orc.i8p),
                                       deltas.ctypes.data_as(orc.f32p), sums.ctypes.data_as(orc.i32p), 1)
        assert rc == -1 and np.all(codes == 17) and np.all(deltas == 19) and np.all(sums == 23)


# ---------------------------------------------------------------- Q8_0 x A8 product order
def test_q8_0_gemv_order_fixture_distinguishes_lane_and_tree_order():
    f = LIT["q8_0_gemv"]["product_order"]
    g = f["groups"]
    w = np.zeros(g * 34, np.uint8)
    w[0::34] = int(f["scale_bits"], 16) & 255
    w[1::34] = int(f["scale_bits"], 16) >> 8
    w[2::34] = f["first_weight_code"]
    codes = np.full((1, g * 32), f["codes_fill"], np.int8)
    deltas = np.zeros((1, g), np.float32)
    for k, v in f["deltas"].items():
        deltas[0, int(k)] = v
    y = np.full((1, 1), f["y_initial"], np.float32)
    orc.gemv_q8_0_a8(w, codes, deltas, g * 32, 1, out=y)
    assert y[0, 0] == f["expect_overwrite"]
    y[:] = f["y_initial"]
    orc.gemv_q8_0_a8(w, codes, deltas, g * 32, 1, out=y, accumulate=True)
    assert y[0, 0] == f["expect_accumulate"]
    # the plain ascending sum gives a different answer, so the fixture really pins the order
    seq = np.float32(0)
    for gi in range(g):
        seq = np.float32(seq + np.float32(32.0) * deltas[0, gi])
    assert seq != np.float32(f["expect_overwrite"])


def test_q8_0_gemv_subnormal_scales_and_padding():
    import ctypes as C
    f = LIT["q8_0_gemv"]["subnormal_scales"]
    w = np.zeros(70, np.uint8)
    w[0] = 1
    w[35], w[36] = 0xFF, 0x83
    w[2:34] = 1
    w[37:69] = 1
    codes = np.full((2, 64), 17, np.int8)
    deltas = np.full((2, 2), 19, np.float32)
    sums = np.full((2, 2), 23, np.int32)
    for r, fb in enumerate(f["x_fill_bits"]):
        x = np.full(32, f32_from_bits(fb), np.float32)
        orc.lib().orc_quantize_a8(x.ctypes.data_as(orc.f32p), C.c_size_t(32), codes[r].ctypes.data_as(orc.i8p),
                                  deltas[r].ctypes.data_as(orc.f32p), sums[r].ctypes.data_as(orc.i32p), 1)
    assert np.all(codes[:, 32:] == 17) and np.all(deltas[:, 1] == 19) and np.all(sums[:, 1] == 23)
    y = np.full((2, 3), 29, np.float32)
    v = orc.Q8a8View(w.ctypes.data, codes.ctypes.data, deltas.ctypes.data, y.ctypes.data, 35, 32, 2, 2, 64, 3, 0)
    assert orc.lib().orc_gemv_q8_0_a8(C.byref(v), 1) == 0
    e = f["expect"]
    assert y[0, 0] == 0 and y[0, 1] == 0
    assert y[1, 0] == np.float32(e["y10_num"]) * np.float32(e["scale"])
    assert y[1, 1] == np.float32(e["y11_num"]) * np.float32(e["scale"])
    assert y[0, 2] == 29 and y[1, 2] == 29


def test_q8_0_gemv_rejects_partial_group_untouched():
    import ctypes as C
    y = np.full((1, 1), 29, np.float32)
    w = np.zeros(68, np.uint8)
    codes = np.zeros((1, 64), np.int8)
    deltas = np.ones((1, 2), np.float32)
    for width in (31, 33):
        v = orc.Q8a8View(w.ctypes.data, codes.ctypes.data, deltas.ctypes.data, y.ctypes.data, 68, width, 1, 1, 64, 1, 0)
        assert orc.lib().orc_gemv_q8_0_a8(C.byref(v), 1) == -1 and y[0, 0] == 29


# ---------------------------------------------------------------- Q4_K x A8 row
def _random_q4k_case(rng, width, headers=None):
    x = np.ldexp((rng.integers(0, 255, width) - 127).astype(np.float32), rng.integers(-8, 7, width).astype(np.int32)).astype(np.float32)
    codes, deltas, sums, _ = orc.quantize_a8(x[None, :], tiny_rule=False)
    w = rng.integers(0, 256, width // 256 * 144, dtype=np.uint8)
    hs = headers or [0, 0x8000, 1, 0x8001, 0x03FF, 0x83FF, 0x3C00, 0xBC00, 0x7BFF, 0xFBFF]
    for b in range(width // 256):
        d, dm = (hs[int(rng.integers(len(hs)))] for _ in range(2))
        w[b * 144:b * 144 + 4] = [d & 255, d >> 8, dm & 255, dm >> 8]
    return w, codes[0], deltas[0], sums[0]


def _py_q4k_row(w, codes, deltas, sums, mutation=None):
    """Independent element-wise evaluation in numpy float32 scalars, with the mutation list of the reference's own
    oracle test (tests/q4k_a8_oracle.hpp:90-127): each mutant must change the bits somewhere."""
    f = np.float32
    acc = [f(-0.0) if mutation == "negative_zero_seed" else f(0.0)] * 4
    nb = codes.size // 256
    for it in range(nb):
        b = nb - 1 - it if mutation == "reverse_blocks" else it
        blk = w[b * 144:(b + 1) * 144]
        d = blk[0:2].copy().view(np.float16)[0].astype(f)
        dm = blk[2:4].copy().view(np.float16)[0].astype(f)
        if mutation == "header_swap":
            d, dm = dm, d
        c = []
        for j in range(8):
            pair = j // 2
            sel = (j ^ 1) if mutation == "nibble_swap" else j
            q = (blk[16 + 32 * pair:16 + 32 * pair + 32].astype(np.int64) >> (4 * (sel & 1))) & 15
            a = codes[b * 256 + j * 32:b * 256 + j * 32 + 32].astype(np.int64)
            if mutation == "unsigned_a":
                a = a & 255
            dot = int((q * a).sum())
            s = int(codes[b * 256 + j * 32:b * 256 + j * 32 + 32].astype(np.int64).sum())
            sc, m = int(orc.lib().orc_q4k_factor_words(blk.ctypes.data_as(orc.u8p), j, 0)), int(orc.lib().orc_q4k_factor_words(blk.ctypes.data_as(orc.u8p), j, 1))
            if mutation == "factor_swap":
                sc, m = m, sc
            i, k = f(sc * dot), f(m * s)
            if mutation == "fused":
                t = f(float(d) * float(i) - float(f(dm * k)))  # one rounding of d*i - RN(dm*k): double is exact enough for 24x24 bits
            else:
                t = f(f(d * i) - f(dm * k))
            c.append(f(deltas[b * 8 + j] * t))
        for p in range(4):
            acc[p] = f(acc[p] + f(c[2 * p] + c[2 * p + 1]))
    if mutation == "missing_xor4":
        return f(acc[0] + acc[1])
    if mutation == "wrong_tree":
        return f(f(acc[0] + acc[2]) + f(acc[1] + acc[3]))
    return f(f(acc[0] + acc[1]) + f(acc[2] + acc[3]))


def test_q4k_row_three_formulations_agree_and_mutants_differ():
    rng = np.random.default_rng(7)
    mutants = ["fused", "reverse_blocks", "wrong_tree", "nibble_swap", "header_swap", "factor_swap", "unsigned_a", "missing_xor4"]
    detected = dict.fromkeys(mutants, False)
    with np.errstate(all="ignore"):
        for width in (256, 512, 2560):
            for _ in range(25):
                w, codes, deltas, sums = _random_q4k_case(rng, width)
                a = orc.q4k_row_a8(w, codes, deltas, sums)
                b = orc.q4k_row_a8(w, codes, deltas, sums, contract_form=True)
                c = _py_q4k_row(w, codes, deltas, sums)
                if np.isnan(c):
                    assert np.isnan(a) and np.isnan(b)
                    continue
                assert bits(a) == bits(b) == bits(c)
                for m in mutants:
                    detected[m] |= bool(bits(_py_q4k_row(w, codes, deltas, sums, m)) != bits(c))
    assert all(detected.values()), detected


def test_q4k_zero_row_is_plus_zero():
    f = LIT["q4k_zero_row"]
    w = np.full(144, f["fill_byte"], np.uint8)
    w[:4] = f["header"]
    codes, deltas, sums, _ = orc.quantize_a8(np.zeros((1, 256), np.float32), tiny_rule=False)
    assert bits(orc.q4k_row_a8(w, codes[0], deltas[0], sums[0])) == int(f["expect_bits"], 16)
    assert bits(_py_q4k_row(w, codes[0], deltas[0], sums[0], "negative_zero_seed")) == 0x80000000


def test_q8_0_down_row_reference_literal_and_chain_order():
    f = LIT["down_rows"]["q8_0"]
    w = np.zeros(f["groups"] * 34, np.uint8)
    w[0::34] = int(f["scale_bits"], 16) & 255
    w[1::34] = int(f["scale_bits"], 16) >> 8
    for g in range(f["groups"]):
        w[g * 34 + 2:(g + 1) * 34] = f["weight_byte"]
    codes = np.full(f["groups"] * 32, f["codes_fill"], np.int8)
    deltas = np.full(f["groups"], f["delta"], np.float32)
    assert orc.q8_0_down_row_a8(w, codes, deltas) == np.float32(f["expect"])
    # cancellation witness for the 4-chain tree: terms 2^30, 1, -2^30, 1 -> (a0+a1)+(a2+a3) = 0, ascending sum = 1
    w2 = np.zeros(4 * 34, np.uint8)
    w2[0::34], w2[1::34] = 0x00, 0x3C
    w2[2::34] = 1
    c2 = np.zeros(128, np.int8)
    c2[0::32] = 1
    d2 = np.array([2.0 ** 30, 1.0, -2.0 ** 30, 1.0], np.float32)
    assert orc.q8_0_down_row_a8(w2, c2, d2) == 0.0


# ---------------------------------------------------------------- exp / SwiGLU
def test_declared_exp_accuracy_and_limits():
    xs = np.linspace(-100, 88, 4001).astype(np.float32)
    got = np.array([orc.lib().orc_declared_exp(float(x)) for x in xs], np.float64)
    want = np.exp(xs.astype(np.float64))
    ok = want > 1e-37
    assert np.max(np.abs(got[ok] / want[ok] - 1)) < 4e-7
    assert orc.lib().orc_declared_exp(89.0) == math.inf and orc.lib().orc_declared_exp(-104.0) == 0.0
    assert orc.lib().orc_declared_exp(0.0) == 1.0


def test_gfx1151_exp_without_tables_is_correctly_rounded_in_range():
    rng = np.random.default_rng(8)
    xs = (rng.uniform(-80, 80, 20000)).astype(np.float32)
    got = np.array([orc.lib().orc_expf_gfx1151(float(x)) for x in xs], np.float32)
    want = np.exp(xs.astype(np.float64))
    # exp2 of the reduced argument is correctly rounded; the reduction adds well under half an ulp
    assert np.max(np.abs(got.astype(np.float64) / want - 1)) < 1.2e-7
    assert orc.lib().orc_expf_gfx1151(-104.0) == 0.0 and orc.lib().orc_expf_gfx1151(89.0) == math.inf


def test_swiglu_quantize_matches_elementwise_definition_and_fails_closed():
    rng = np.random.default_rng(9)
    g = rng.standard_normal(32).astype(np.float32) * 3
    u = rng.standard_normal(32).astype(np.float32) * 3
    ok, codes, delta, s, h = orc.swiglu_quantize(g, u)
    f = np.float32
    hv = np.array([f(f(g[i] / f(f(1.0) + f(orc.lib().orc_expf_gfx1151(float(-g[i]))))) * u[i]) for i in range(32)], np.float32)
    assert ok == 1 and np.array_equal(bits(h), bits(hv))
    c2, d2, s2, _ = orc.quantize_a8(hv[None, :], tiny_rule=True)
    assert np.array_equal(codes, c2[0]) and bits(delta) == bits(d2[0, 0]) and s == s2[0, 0]
    g[5] = np.inf
    ok, codes, *_ = orc.swiglu_quantize(g, u)
    assert ok == 0 and np.all(codes == 0)


# ---------------------------------------------------------------- router
def test_router_selection_equals_stable_sort_and_weight_bits():
    rng = np.random.default_rng(10)
    for experts, top_k in ((128, 8), (256, 8), (160, 8), (64, 1)):
        for _ in range(20):
            z = (rng.integers(-512, 513, experts) / 64.0).astype(np.float32)  # 1/64 grid: exact ties
            m = z.max()
            p = np.array([orc.lib().orc_declared_exp(float(np.float32(v - m))) for v in z], np.float32)
            tot = np.float32(0)
            for v in p:
                tot = np.float32(tot + v)
            s = (p / tot).astype(np.float32)
            ids, w = orc.route_select(s, top_k, renorm_eps=1e-20, scale=2.5)
            want = sorted(range(experts), key=lambda e: (-s[e], e))[:top_k]
            assert list(ids) == want
            acc = np.float32(0)
            for e in ids:
                acc = np.float32(acc + s[e])
            den = np.float32(acc + np.float32(1e-20))
            for k, e in enumerate(ids):
                assert bits(w[k]) == bits(np.float32(np.float32(s[e] / den) * np.float32(2.5)))
    s = np.full(16, 0.25, np.float32)
    ids, _ = orc.route_select(s, 4)
    assert list(ids) == [0, 1, 2, 3]


def test_router_logit_chains_softmax_and_bias():
    rng = np.random.default_rng(11)
    x = rng.standard_normal((3, 96)).astype(np.float32)
    w = (rng.standard_normal((16, 96)) * 0.02).astype(np.float32)
    bias = rng.standard_normal(16).astype(np.float32)
    ids, wt, scores, logits = orc.route(x, w, 4, bias=bias)
    for r in range(3):
        for e in range(16):
            acc = 0.0
            for k in range(96):  # fma in double then one rounding == fmaf for 24-bit operands
                acc = float(np.float32(float(x[r, k]) * float(w[e, k]) + acc))
            assert bits(logits[r, e]) == bits(np.float32(np.float32(acc) + bias[e]))
        assert abs(float(scores[r].sum()) - 1) < 1e-5
        assert list(ids[r]) == sorted(range(16), key=lambda e: (-scores[r, e], e))[:4]
    _, _, _, lg2 = orc.route(x, w, 4, logits_order=orc.LOGITS_LANE32)
    for r in range(3):
        for e in range(16):
            assert bits(lg2[r, e]) == bits(np.float32(orc.lib().orc_lane_dot((w[e] * 1).ctypes.data_as(orc.f32p), x[r].ctypes.data_as(orc.f32p), 96)))
    assert np.max(np.abs(lg2 - (logits - bias))) < 1e-5


# ---------------------------------------------------------------- combine
def test_combine_forms_and_commit_threshold():
    rng = np.random.default_rng(12)
    raw = rng.standard_normal((2, 4, 8)).astype(np.float32)
    w = rng.random((2, 4)).astype(np.float32)
    ids = np.array([[7, 2, 9, 0], [1, 5, 3, 4]], np.uint32)
    base = rng.standard_normal((2, 8)).astype(np.float32)
    y = orc.combine(orc.COMBINE_FMA_SLOT, w, ids, raw, base)
    z = orc.combine(orc.COMBINE_MULADD_ASC, w, ids, raw)
    for r in range(2):
        for d in range(8):
            acc = np.float32(0)
            for k in range(4):
                acc = np.float32(float(w[r, k]) * float(raw[r, k, d]) + float(acc))
            assert bits(y[r, d]) == bits(np.float32(acc + base[r, d]))
            s = np.float32(0)
            for k in np.argsort(ids[r], kind="stable"):
                s = np.float32(s + np.float32(w[r, k] * raw[r, k, d]))
            assert bits(z[r, d]) == bits(s)
    assert int(LIT["commit_threshold"]["bf16_bits"], 16) == 0x7F7F8000


# ---------------------------------------------------------------- whole layer, brute force on tiny shapes
def _tiny_layer(rng, H, I, E, T, K, down_type):
    gate = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((E, I, H)) * 0.05).astype(np.float32))
    up = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((E, I, H)) * 0.05).astype(np.float32))
    if down_type == orc.Q5_1:
        down = orc.random_q5_1(rng, (E, H), I)
    else:
        down = orc.quantize_rows(down_type, (rng.standard_normal((E, H, I)) * 0.05).astype(np.float32))
    x = rng.standard_normal((T, H)).astype(np.float16).astype(np.float32)
    ids = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.uint32)
    return gate, up, down, x, ids


@pytest.mark.parametrize("down_type", [orc.Q4_K, orc.Q8_0, orc.Q5_1])
def test_routed_experts_against_double_precision_dequant_reference(down_type):
    """Brute force: A8-quantise explicitly, dequantise weights with the (separately pinned) block decoders, sum in
    double. The declared fp32 chain must agree to fp32 accumulation accuracy; a dropped term or a wrong index is O(1)."""
    rng = np.random.default_rng(13)
    H, I, E, T, K = 512, 256, 6, 3, 2
    gate, up, down, x, ids = _tiny_layer(rng, H, I, E, T, K, down_type)
    codes, deltas, sums, _ = orc.quantize_a8(x)
    r = orc.routed_experts(H, I, K, gate, up, down, down_type, codes, deltas, sums, ids)
    assert r.bad == 0 and np.all(r.status == 0)
    xa = (codes.astype(np.float64) * np.repeat(deltas.astype(np.float64), 32, axis=1))
    for t in range(T):
        for k in range(K):
            e = ids[t, k]
            a = t * K + k
            G = orc.dequant_rows(orc.Q4_K, gate[e], H).astype(np.float64) @ xa[t]
            U = orc.dequant_rows(orc.Q4_K, up[e], H).astype(np.float64) @ xa[t]
            assert np.max(np.abs(r.gate[a] - G)) < 2e-5 * max(1, np.abs(G).max())
            assert np.max(np.abs(r.up[a] - U)) < 2e-5 * max(1, np.abs(U).max())
            ha = r.h_codes[a].astype(np.float64) * np.repeat(r.h_deltas[a].astype(np.float64), 32)
            hd = r.gate[a].astype(np.float64) / (1 + np.exp(-r.gate[a].astype(np.float64))) * r.up[a].astype(np.float64)
            assert np.max(np.abs(ha - hd)) <= np.abs(hd).reshape(-1, 32).max(-1).repeat(32).max() / 127 * 0.51 + 1e-9
            wd = orc.dequant_q5_1_rows(down[e], I) if down_type == orc.Q5_1 else orc.dequant_rows(down_type, down[e], I)
            D = wd.astype(np.float64) @ ha
            assert np.max(np.abs(r.rawdots[t, k] - D)) < 2e-5 * max(1, np.abs(D).max())
    # the down phase alone, from the same h image, gives the same bits (stage-by-stage form used by the GPU tests)
    r2 = orc.routed_experts(H, I, K, gate, up, down, down_type, codes, deltas, sums, ids, down_only_from=(r.h_codes, r.h_deltas, r.h_sums))
    assert np.array_equal(bits(r2.rawdots), bits(r.rawdots))
    # thread count never changes a bit
    r1 = orc.routed_experts(H, I, K, gate, up, down, down_type, codes, deltas, sums, ids, threads=1)
    assert np.array_equal(bits(r1.rawdots), bits(r.rawdots)) and np.array_equal(r1.h_codes, r.h_codes)


def test_q5k_test_writer_round_trip():
    """The tests' own Q5_K writer: decoding what it wrote returns the input to within half a code step, and the fifth bits are
    in use (codes above 15 exist)."""
    rng = np.random.default_rng(17)
    x = (rng.standard_normal((6, 1024)) * 0.02).astype(np.float32)
    packed = orc.quantize_q5_k_rows(x)
    assert packed.shape == (6, 4 * 176) and packed.reshape(6, 4, 176)[..., 16:48].any()
    back = orc.dequant_q5_k_rows(packed, 1024)
    step = (x.reshape(6, 4, 8, 32).max(-1) - np.minimum(x.reshape(6, 4, 8, 32).min(-1), 0)) / 31
    assert np.max(np.abs(back - x).reshape(6, 4, 8, 32) / (step[..., None] + 1e-12)) < 1.6


def test_q5k_gate_rows_against_double_precision_dequant_reference():
    """Brute force for the Q5_K gate/up row: dequantise with a numpy statement of the block layout, sum in double."""
    rng = np.random.default_rng(15)
    H = 768
    w = orc.random_q5_k(rng, (40,), H)
    x = rng.standard_normal((3, H)).astype(np.float32)
    codes, deltas, sums, _ = orc.quantize_a8(x)
    xa = codes.astype(np.float64) * np.repeat(deltas.astype(np.float64), 32, axis=1)
    want = xa @ orc.dequant_q5_k_rows(w, H).astype(np.float64).T
    got = np.array([[orc.q5k_row_a8(w[o], codes[t], deltas[t], sums[t]) for o in range(40)] for t in range(3)])
    assert np.max(np.abs(got - want)) < 2e-5 * np.abs(want).max()
    # the fifth bits matter: clearing them changes every row
    w4 = w.copy().reshape(40, -1, 176)
    w4[..., 16:48] = 0
    assert np.all(np.array([orc.q5k_row_a8(w4[o].reshape(-1), codes[0], deltas[0], sums[0]) for o in range(40)]) != got[0])


def test_q6k_down_rows_against_the_contract_and_double_precision():
    """Q6_K down row: bitwise against the compiled reference's contract oracle (evaluate_down_row, type 14) where it is built,
    and against a float64 sum over a numpy statement of the block layout."""
    import ctypes as C
    rng = np.random.default_rng(16)
    for width in (256, 768, 1280, 1536):                     # the contract oracle admits K-quant rows up to 1536
        w = orc.random_q6_k(rng, (12,), width)
        x = (rng.standard_normal((2, width)) * 3.0).astype(np.float32)
        codes, deltas, sums, _ = orc.quantize_a8(x, tiny_rule=True)
        got = np.array([[orc.q6k_down_row_a8(w[o], codes[t], deltas[t]) for o in range(12)] for t in range(2)])
        xa = codes.astype(np.float64) * np.repeat(deltas.astype(np.float64), 32, axis=1)
        want = xa @ orc.dequant_q6_k_rows(w, width).astype(np.float64).T
        assert np.max(np.abs(got - want)) < 2e-5 * np.abs(want).max()
        R = orc.ref()
        if R is not None:
            out = C.c_float(0)
            for t in range(2):
                for o in range(12):
                    assert R.ref_evaluate_down_row(w[o].ctypes.data_as(orc.u8p), C.c_size_t(w[o].size), codes[t].ctypes.data_as(orc.i8p),
                                                   deltas[t].ctypes.data_as(orc.f32p), sums[t].ctypes.data_as(orc.i32p), C.c_size_t(width), 14,
                                                   C.byref(out)) == 0, R.ref_last_error()
                    assert bits(np.float32(got[t, o])) == bits(np.float32(out.value))


def test_routed_experts_nonfinite_row_sets_status_and_skips_down():
    rng = np.random.default_rng(14)
    H, I, E, T, K = 256, 128, 3, 2, 2
    gate, up, down, x, ids = _tiny_layer(rng, H, I, E, T, K, orc.Q8_0)
    codes, deltas, sums, _ = orc.quantize_a8(x)
    deltas[1, 3] = 3.0e38  # the host-forceable failure of tests/cpu/routed_expert_host_tests.cpp:393-406
    r = orc.routed_experts(H, I, K, gate, up, down, orc.Q8_0, codes, deltas, sums, ids)
    assert r.bad == 1 and r.status[0] == 0 and r.status[1] & 8
    assert np.all(r.rawdots == 0)


def test_tp_rank_partials_tile_the_unsplit_expert():
    """Expert tensor-parallel split by the intermediate dimension: each rank's gate/up rows and h groups are exactly
    the unsplit expert's (whole 32-groups move), and the two rank partials sum to the unsplit down product up to fp32
    reassociation (the split is its own arithmetic identity: include/strix/ds41_expert_tp.hpp:3-19)."""
    rng = np.random.default_rng(15)
    H, I, E, T, K = 512, 512, 4, 2, 2
    gate, up, down, x, ids = _tiny_layer(rng, H, I, E, T, K, orc.Q4_K)
    codes, deltas, sums, _ = orc.quantize_a8(x)
    full = orc.routed_experts(H, I, K, gate, up, down, orc.Q4_K, codes, deltas, sums, ids)
    half = I // 2
    grb, drb = H // 256 * 144, I // 256 * 144
    parts = []
    for rank in range(2):
        g = gate.reshape(-1)[rank * half * grb:]
        u = up.reshape(-1)[rank * half * grb:]
        d = down.reshape(-1)[rank * (half // 256) * 144:]
        p = orc.routed_experts(H, half, K, g, u, d, orc.Q4_K, codes, deltas, sums, ids, gate_expert_stride=I * grb,
                               gate_row_stride=grb, down_expert_stride=H * drb, down_row_stride=drb)
        assert np.array_equal(p.h_codes, full.h_codes[:, rank * half:(rank + 1) * half])
        assert np.array_equal(bits(p.h_deltas), bits(full.h_deltas[:, rank * half // 32:(rank + 1) * half // 32]))
        assert np.array_equal(bits(p.gate), bits(full.gate[:, rank * half:(rank + 1) * half]))
        parts.append(p.rawdots)
    total = parts[0].astype(np.float64) + parts[1].astype(np.float64)
    assert np.max(np.abs(total - full.rawdots)) < 1e-5 * np.abs(full.rawdots).max()
    assert not np.array_equal(bits(parts[0]), bits(full.rawdots))


def test_base_linear_matches_numpy_double():
    rng = np.random.default_rng(16)
    wq = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((8, 512)) * 0.02).astype(np.float32))
    x = rng.standard_normal((3, 512)).astype(np.float16).astype(np.float32)
    y = orc.base_linear(orc.Q4_K, wq, 2 * 144, 8, 512, x)
    want = x.astype(np.float64) @ orc.dequant_rows(orc.Q4_K, wq, 512).astype(np.float64).T
    assert np.array_equal(bits(y), bits(want.astype(np.float32)))


# ---------------------------------------------------------------- bitwise against the compiled reference
needs_ref = pytest.mark.skipif(orc.ref() is None, reason="oracle/_ref not built (no reference tree at build time)")


@needs_ref
def test_ref_half_and_dequant_bits():
    import ctypes as C
    R = orc.ref()
    for h in range(0, 65536, 1):
        a, b = orc.half_to_float(h), R.ref_half_to_float(C.c_uint16(h))
        assert (math.isnan(a) and math.isnan(b)) or bits(a) == bits(b)
    rng = np.random.default_rng(20)
    for qtype, rb, n in ((orc.Q8_0, 34 * 8, 256), (orc.Q4_K, 144 * 2, 512)):
        raw = rng.integers(0, 256, (16, rb), dtype=np.uint8)
        mine = orc.dequant_rows(qtype, raw, n)
        theirs = np.zeros_like(mine)
        for r in range(16):
            assert R.ref_dequantize_row(qtype, raw[r].ctypes.data_as(orc.u8p), C.c_size_t(rb), theirs[r].ctypes.data_as(orc.f32p), C.c_size_t(n)) == 0
        assert np.array_equal(bits(mine), bits(theirs))


@needs_ref
def test_ref_a8_and_q8_0_gemv_bits():
    import ctypes as C
    R = orc.ref()
    rng = np.random.default_rng(21)
    x = rng.standard_normal((4, 1024)).astype(np.float32)
    x[1, :32] = 0
    x[2, 32:64] = 1e-37
    codes, deltas, sums, _ = orc.quantize_a8(x, tiny_rule=True)
    c2, d2, s2 = np.zeros_like(codes), np.zeros_like(deltas), np.zeros_like(sums)
    for r in range(4):
        assert R.ref_quantize_a8(x[r].ctypes.data_as(orc.f32p), C.c_size_t(1024), c2[r].ctypes.data_as(orc.i8p),
                                 d2[r].ctypes.data_as(orc.f32p), s2[r].ctypes.data_as(orc.i32p)) == 0
    assert np.array_equal(codes, c2) and np.array_equal(bits(deltas), bits(d2)) and np.array_equal(sums, s2)
    w = orc.quantize_rows(orc.Q8_0, (rng.standard_normal((96, 1024)) * 0.02).astype(np.float32))
    y, rc = orc.gemv_q8_0_a8(w, codes, deltas, 1024, 96, threads=3)
    y2 = np.zeros_like(y)
    v = orc.Q8a8View(w.ctypes.data, codes.ctypes.data, deltas.ctypes.data, y2.ctypes.data, 1024 // 32 * 34, 1024, 96, 4, 1024, 96, 0)
    assert R.ref_gemv_q8_0_a8(C.byref(v)) == 0
    assert np.array_equal(bits(y), bits(y2))


@needs_ref
def test_ref_q4k_row_and_down_row_bits_at_config_widths():
    import ctypes as C
    R = orc.ref()
    rng = np.random.default_rng(22)
    out = C.c_float(0)
    for width in (256, 2048, 768, 1280, 2560):   # contract oracle caps: hidden <= 2560
        for _ in range(8):
            x = (rng.standard_normal(width) * rng.choice([1e-3, 1.0, 30.0])).astype(np.float32)
            codes, deltas, sums, _ = orc.quantize_a8(x[None, :], tiny_rule=False)
            w = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((1, width)) * 0.02).astype(np.float32))[0]
            mine = orc.q4k_row_a8(w, codes[0], deltas[0], sums[0])
            assert R.ref_q4k_evaluate_row(w.ctypes.data_as(orc.u8p), C.c_size_t(w.size), codes[0].ctypes.data_as(orc.i8p),
                                          deltas[0].ctypes.data_as(orc.f32p), sums[0].ctypes.data_as(orc.i32p), C.c_size_t(width), C.byref(out)) == 0, R.ref_last_error()
            assert bits(mine) == bits(np.float32(out.value))
    for width in (5120, 27648, 4096, 6144):       # the host executor's row kernel has no cap
        x = rng.standard_normal(width).astype(np.float32)
        codes, deltas, sums, _ = orc.quantize_a8(x[None, :])
        w = rng.integers(0, 256, width // 256 * 144, dtype=np.uint8)
        w[1::144] = (w[1::144] & 0x03) | 0x10
        w[3::144] = (w[3::144] & 0x03) | 0x10
        R.ref_gate_row_q4k(w.ctypes.data_as(orc.u8p), width // 256, codes[0].ctypes.data_as(orc.i8p), deltas[0].ctypes.data_as(orc.f32p),
                           sums[0].ctypes.data_as(orc.i32p), C.byref(out))
        assert bits(orc.q4k_row_a8(w, codes[0], deltas[0], sums[0])) == bits(np.float32(out.value))
        w8 = orc.quantize_rows(orc.Q8_0, (rng.standard_normal((1, width)) * 0.02).astype(np.float32))[0]
        R.ref_down_row_q8_0(w8.ctypes.data_as(orc.u8p), width // 32, codes[0].ctypes.data_as(orc.i8p), deltas[0].ctypes.data_as(orc.f32p),
                            sums[0].ctypes.data_as(orc.i32p), C.byref(out))
        assert bits(orc.q8_0_down_row_a8(w8, codes[0], deltas[0])) == bits(np.float32(out.value))
        wk = orc.random_q5_k(rng, (1,), width)[0]
        R.ref_gate_row_q5k(wk.ctypes.data_as(orc.u8p), width // 256, codes[0].ctypes.data_as(orc.i8p), deltas[0].ctypes.data_as(orc.f32p),
                           sums[0].ctypes.data_as(orc.i32p), C.byref(out))
        assert bits(orc.q5k_row_a8(wk, codes[0], deltas[0], sums[0])) == bits(np.float32(out.value))
        w5 = orc.random_q5_1(rng, (1,), width)[0]
        R.ref_down_row_q5_1(w5.ctypes.data_as(orc.u8p), width // 32, codes[0].ctypes.data_as(orc.i8p), deltas[0].ctypes.data_as(orc.f32p),
                            sums[0].ctypes.data_as(orc.i32p), C.byref(out))
        assert bits(orc.q5_1_down_row_a8(w5, codes[0], deltas[0], sums[0])) == bits(np.float32(out.value))


@needs_ref
def test_ref_rmsnorm_bits():
    """RMSNorm (lane-strided fma chains, halving tree): the restatement against the compiled reference kernel table, bit for
    bit, for both lane counts, with and without the weight vector; and against float64 to 1e-6."""
    import ctypes as C
    R = orc.ref()
    rng = np.random.default_rng(27)
    for n, rows in ((64, 3), (511, 2), (512, 2), (2048, 4), (5120, 2), (6144, 1)):
        x = (rng.standard_normal((rows, n)) * rng.choice([1e-3, 1.0, 50.0])).astype(np.float32)
        w = rng.standard_normal(n).astype(np.float32)
        for weight in (w, None):
            mine = orc.rmsnorm_f32(x, weight, 1e-6)
            theirs = np.empty_like(x)
            wp = None if weight is None else weight.ctypes.data_as(orc.f32p)
            assert R.ref_rmsnorm_f32(x.ctypes.data_as(orc.f32p), wp, n, C.c_float(1e-6), theirs.ctypes.data_as(orc.f32p), rows) == 0, R.ref_last_error()
            assert np.array_equal(bits(mine), bits(theirs))
            x64 = x.astype(np.float64)
            want = x64 / np.sqrt(np.mean(x64 ** 2, axis=1, keepdims=True) + 1e-6) * (1.0 if weight is None else weight.astype(np.float64))
            assert np.max(np.abs(mine - want)) <= 2e-6 * np.max(np.abs(want))


@needs_ref
def test_ref_exp_functions_bits():
    R = orc.ref()
    rng = np.random.default_rng(23)
    xs = np.concatenate([rng.uniform(-110, 95, 40000), rng.standard_normal(40000) * 4, [0.0, -0.0, 88.0, -103.0, 88.7, -104.0]]).astype(np.float32)
    for x in xs:
        assert bits(orc.lib().orc_declared_exp(float(x))) == bits(R.ref_declared_exp(float(x)))
        assert bits(orc.lib().orc_expf_gfx1151(float(x))) == bits(R.ref_gfx1151_expf_empty_tables(float(x)))


@needs_ref
def test_ref_whole_routed_expert_job_bits():
    """reference_run and the pooled executor (scalar and AVX2 tables) against the restated layer: Q4_K gate/up, Q8_0 down."""
    import ctypes as C
    R = orc.ref()
    rng = np.random.default_rng(24)
    H, I, E, T, K = 512, 256, 6, 5, 3
    gate, up, down, x, ids = _tiny_layer(rng, H, I, E, T, K, orc.Q8_0)
    codes, deltas, sums, _ = orc.quantize_a8(x)
    mine = orc.routed_experts(H, I, K, gate, up, down, orc.Q8_0, codes, deltas, sums, ids)
    asg = np.array([[t, k, ids[t, k]] for t in range(T) for k in range(K)], np.uint32)
    for threads, simd in ((0, 0), (1, 0), (3, 1), (8, 1)):
        raw = np.zeros((T, K, H), np.float32)
        status = np.zeros(T, np.uint32)
        rc = R.ref_routed_expert_run(H, I, gate.ctypes.data_as(orc.u8p), up.ctypes.data_as(orc.u8p), down.ctypes.data_as(orc.u8p),
                                     codes.ctypes.data_as(orc.i8p), deltas.ctypes.data_as(orc.f32p), sums.ctypes.data_as(orc.i32p), T,
                                     asg.ctypes.data_as(orc.u32p), T * K, raw.ctypes.data_as(orc.f32p), C.c_uint64(K * H),
                                     status.ctypes.data_as(orc.u32p), threads, simd)
        assert rc == 0, R.ref_last_error()
        assert np.array_equal(bits(raw), bits(mine.rawdots)) and np.all(status == 0)
    # the executor's other down format: Q5_1 (random blocks: the reference has no writer for it either)
    down5 = orc.random_q5_1(rng, (E, H), I)
    mine5 = orc.routed_experts(H, I, K, gate, up, down5, orc.Q5_1, codes, deltas, sums, ids)
    assert not np.array_equal(bits(mine5.rawdots), bits(mine.rawdots))
    for threads, simd in ((0, 0), (3, 1)):
        raw = np.zeros((T, K, H), np.float32)
        status = np.zeros(T, np.uint32)
        rc = R.ref_routed_expert_run_fmt(H, I, gate.ctypes.data_as(orc.u8p), up.ctypes.data_as(orc.u8p), down5.ctypes.data_as(orc.u8p), 1,
                                         codes.ctypes.data_as(orc.i8p), deltas.ctypes.data_as(orc.f32p), sums.ctypes.data_as(orc.i32p), T,
                                         asg.ctypes.data_as(orc.u32p), T * K, raw.ctypes.data_as(orc.f32p), C.c_uint64(K * H),
                                         status.ctypes.data_as(orc.u32p), threads, simd)
        assert rc == 0, R.ref_last_error()
        assert np.array_equal(bits(raw), bits(mine5.rawdots)) and np.all(status == 0)
    # the executor's other gate/up format: Q5_K (random blocks), with either down format
    gate5, up5 = orc.random_q5_k(rng, (E, I), H), orc.random_q5_k(rng, (E, I), H)
    for down_t, down_w, flags in ((orc.Q8_0, down, 2), (orc.Q5_1, down5, 3)):
        mine_k = orc.routed_experts(H, I, K, gate5, up5, down_w, down_t, codes, deltas, sums, ids, gate_type=orc.Q5_K)
        for threads, simd in ((0, 0), (3, 1)):
            raw = np.zeros((T, K, H), np.float32)
            status = np.zeros(T, np.uint32)
            rc = R.ref_routed_expert_run_fmt(H, I, gate5.ctypes.data_as(orc.u8p), up5.ctypes.data_as(orc.u8p), down_w.ctypes.data_as(orc.u8p), flags,
                                             codes.ctypes.data_as(orc.i8p), deltas.ctypes.data_as(orc.f32p), sums.ctypes.data_as(orc.i32p), T,
                                             asg.ctypes.data_as(orc.u32p), T * K, raw.ctypes.data_as(orc.f32p), C.c_uint64(K * H),
                                             status.ctypes.data_as(orc.u32p), threads, simd)
            assert rc == 0, R.ref_last_error()
            assert np.array_equal(bits(raw), bits(mine_k.rawdots)) and np.all(status == 0)


@needs_ref
def test_ref_router_policy_and_combine_bits():
    import ctypes as C
    R = orc.ref()
    rng = np.random.default_rng(25)
    for experts, top_k in ((128, 8), (256, 8), (160, 8)):
        z = (rng.standard_normal(experts) * 0.9).astype(np.float32)
        z[5] = z[17]  # an exact tie
        s_ref = np.zeros(experts, np.float32)
        assert R.ref_route_scores_softmax(z.ctypes.data_as(orc.f32p), C.c_size_t(experts), s_ref.ctypes.data_as(orc.f32p), 0) == 0
        x = np.zeros((1, 1), np.float32)
        # drive the oracle's softmax with the same logits: hidden 1, x = 1, w = z  (fma(1, z, 0) = z)
        ids, w, scores, logits = orc.route(np.ones((1, 1), np.float32), z[:, None].copy(), top_k, renorm_eps=0.0)
        assert np.array_equal(bits(scores[0]), bits(s_ref))
        ids_ref, w_ref = np.zeros(top_k, np.uint32), np.zeros(top_k, np.float32)
        assert R.ref_route_select(experts, top_k, C.c_float(0.0), C.c_float(1.0), 1, s_ref.ctypes.data_as(orc.f32p),
                                  ids_ref.ctypes.data_as(orc.u32p), w_ref.ctypes.data_as(orc.f32p)) == 0
        assert np.array_equal(ids[0], ids_ref) and np.array_equal(bits(w[0]), bits(w_ref))
    raw = rng.standard_normal((3, 8, 64)).astype(np.float32)
    w = rng.random((3, 8)).astype(np.float32)
    base = rng.standard_normal((3, 64)).astype(np.float32)
    y_ref = np.zeros((3, 64), np.float32)
    assert R.ref_combine_fma(3, 8, 64, w.ctypes.data_as(orc.f32p), raw.ctypes.data_as(orc.f32p), base.ctypes.data_as(orc.f32p),
                             y_ref.ctypes.data_as(orc.f32p)) == 0
    y = orc.combine(orc.COMBINE_FMA_SLOT, w, np.zeros((3, 8), np.uint32), raw, base)
    assert np.array_equal(bits(y), bits(y_ref))
    for has_w, has_base in ((True, True), (True, False), (False, True), (False, False)):         # CombineForm::bf16_steps
        p = lambda a, on: a.ctypes.data_as(orc.f32p) if on else None
        assert R.ref_combine_bf16_steps(3, 8, 64, p(w, has_w), p(raw, True), p(base, has_base), p(y_ref, True)) == 0
        y = orc.combine(orc.COMBINE_BF16_STEPS, w if has_w else None, None, raw, base if has_base else None)
        assert np.array_equal(bits(y), bits(y_ref)), (has_w, has_base)


@needs_ref
def test_ref_router_libm_exp_scores_and_single_expert_renormalisation():
    """Math::exp = the C library's expf (the reference's router test oracle) and the policy's renorm_single field, both
    against the compiled reference policy functions."""
    import ctypes as C
    R = orc.ref()
    rng = np.random.default_rng(31)
    for experts in (128, 257):
        z = (rng.standard_normal(experts) * 2.5).astype(np.float32)
        s_ref = np.zeros(experts, np.float32)
        assert R.ref_route_scores_softmax(z.ctypes.data_as(orc.f32p), C.c_size_t(experts), s_ref.ctypes.data_as(orc.f32p), 1) == 0
        _, _, scores, _ = orc.route(np.ones((1, 1), np.float32), z[:, None].copy(), 4, exp_kind=orc.EXP_LIBM)
        assert np.array_equal(bits(scores[0]), bits(s_ref))
        _, _, declared, _ = orc.route(np.ones((1, 1), np.float32), z[:, None].copy(), 4, exp_kind=orc.EXP_DECLARED)
        assert not np.array_equal(bits(declared[0]), bits(s_ref))          # the two Math traits differ in bits
        for top_k in (1, 2):
            for renormalize in (0, 1):
                for single in (0, 1):
                    ids_ref, w_ref = np.zeros(top_k, np.uint32), np.zeros(top_k, np.float32)
                    assert R.ref_route_select_policy(experts, top_k, C.c_float(1e-20), C.c_float(2.5), renormalize, single,
                                                     s_ref.ctypes.data_as(orc.f32p), ids_ref.ctypes.data_as(orc.u32p),
                                                     w_ref.ctypes.data_as(orc.f32p)) == 0
                    ids, w = orc.route_select(s_ref, top_k, renorm_eps=1e-20, scale=2.5, renormalize=bool(renormalize), renorm_single=bool(single))
                    assert np.array_equal(ids, ids_ref) and np.array_equal(bits(w), bits(w_ref)), (top_k, renormalize, single)
    # top_k = 1: the weight is s * scale unless renorm_single is set (then s / (s + eps) * scale)
    ids, w = orc.route_select(s_ref, 1, renorm_eps=0.0, scale=2.0, renormalize=True, renorm_single=False)
    assert bits(w)[0] == bits(np.float32(s_ref[ids[0]] * np.float32(2.0)))
    ids, w = orc.route_select(s_ref, 1, renorm_eps=0.0, scale=2.0, renormalize=True, renorm_single=True)
    assert w[0] == np.float32(2.0)


def libm_expf_restated(x):
    """The algorithm the device uses for Math::exp = expf (csrc/device_math.hpp expf_libm), in numpy double precision."""
    import struct
    tab = np.array([struct.unpack("<Q", struct.pack("<d", 2.0 ** (i / 32.0)))[0] - (i << 47) for i in range(32)], np.uint64)
    xd = x.astype(np.float64)
    z = (float.fromhex("0x1.71547652b82fep+0") * 32.0) * xd
    kd = z + float.fromhex("0x1.8p+52")
    ki = kd.view(np.uint64)
    kd = kd - float.fromhex("0x1.8p+52")
    r = z - kd
    s = (tab[(ki % np.uint64(32)).astype(np.int64)] + (ki << np.uint64(47))).view(np.float64)
    c01 = (float.fromhex("0x1.c6af84b912394p-5") / 32.0 / 32.0 / 32.0) * r + (float.fromhex("0x1.ebfce50fac4f3p-3") / 32.0 / 32.0)
    y = (float.fromhex("0x1.62e42ff0c52d6p-1") / 32.0) * r + 1.0
    y = c01 * (r * r) + y
    return (y * s).astype(np.float32)


def test_libm_expf_restatement_equals_the_c_library():
    """Two million arguments over the softmax range (x <= 0) and beyond: the table-and-cubic algorithm in double precision
    gives the C library's bits (the table entries are the correctly rounded 2^(i/32), checked against Python's pow here)."""
    import ctypes as C
    libm = C.CDLL("libm.so.6")
    libm.expf.restype, libm.expf.argtypes = C.c_float, [C.c_float]
    rng = np.random.default_rng(41)
    x = np.concatenate([-rng.random(1_200_000) * 40.0, rng.standard_normal(500_000) * 6.0, rng.uniform(-87.0, 88.0, 300_000)]).astype(np.float32)
    got = libm_expf_restated(x)
    sample = rng.choice(x.size, 60_000, replace=False)
    want = np.array([libm.expf(float(v)) for v in x[sample]], np.float32)
    assert np.array_equal(bits(got[sample]), bits(want))
    # the oracle's EXP_LIBM softmax is that function: one-expert-hot rows give exp(z - max) / sum directly
    z = np.array([0.0, -1.5, -7.25, -30.0], np.float32)
    _, _, scores, _ = orc.route(np.ones((1, 1), np.float32), z[:, None].copy(), 1, exp_kind=orc.EXP_LIBM)
    p = libm_expf_restated(z)
    total = np.float32(0.0)
    for v in p:
        total = np.float32(total + v)
    assert np.array_equal(bits(scores[0]), bits((p / total).astype(np.float32)))


def test_swiglu_clamp_trait():
    """The clamp acts on the projections before silu(g) * u (gate from above only, up on both sides), a huge limit is no
    clamp bit for bit, and the fail-closed check stays on the RAW projections (an infinite gate that the clamp would hide
    still fails)."""
    rng = np.random.default_rng(43)
    g = (rng.standard_normal(32) * 6.0).astype(np.float32)
    u = (rng.standard_normal(32) * 6.0).astype(np.float32)
    L = 2.5
    for kind in (orc.EXP_GFX1151, orc.EXP_DECLARED):
        plain = orc.swiglu_quantize(g, u, kind)
        huge = orc.swiglu_quantize(g, u, kind, limit=1e30)
        assert huge[0] == plain[0] == 1 and np.array_equal(huge[1], plain[1]) and bits(huge[2]) == bits(plain[2]) and np.array_equal(bits(huge[4]), bits(plain[4]))
        clamped = orc.swiglu_quantize(g, u, kind, limit=L)
        by_hand = orc.swiglu_quantize(np.minimum(g, np.float32(L)), np.clip(u, -np.float32(L), np.float32(L)), kind)
        assert np.array_equal(clamped[1], by_hand[1]) and bits(clamped[2]) == bits(by_hand[2]) and clamped[3] == by_hand[3]
        assert np.array_equal(bits(clamped[4]), bits(by_hand[4])) and not np.array_equal(clamped[1], plain[1])
        low = g.copy(); low[3] = -40.0          # the gate is not clamped from below
        assert orc.swiglu_quantize(low, u, kind, limit=L)[4][3] == orc.swiglu_quantize(low, np.clip(u, -L, L).astype(np.float32), kind)[4][3]
        bad = g.copy(); bad[7] = np.inf
        assert orc.swiglu_quantize(bad, u, kind, limit=L)[0] == 0
    R = orc.ref()
    if R is not None:
        import ctypes as C
        R.ref_swiglu_clamp.argtypes = [C.c_float, C.c_float, C.c_float, C.POINTER(C.c_float), C.POINTER(C.c_float)]
        for gv, uv in ((3.0, -9.0), (-8.0, 9.0), (float("nan"), 1.0), (1.0, float("nan")), (2.5, 2.5), (float("inf"), float("-inf"))):
            a, b = C.c_float(0), C.c_float(0)
            R.ref_swiglu_clamp(gv, uv, L, C.byref(a), C.byref(b))
            want_g = gv if not gv > L else L
            want_u = -L if uv < -L else (L if uv > L else uv)
            assert (math.isnan(a.value) and math.isnan(want_g)) or a.value == want_g
            assert (math.isnan(b.value) and math.isnan(want_u)) or b.value == want_u
            # and the oracle applies exactly that pair: h of a one-value group
            gg, uu = np.zeros(32, np.float32), np.zeros(32, np.float32)
            gg[0], uu[0] = gv, uv
            ok, _, _, _, h = orc.swiglu_quantize(gg, uu, orc.EXP_DECLARED, limit=L)
            if math.isfinite(gv) and math.isfinite(uv):
                hh = orc.swiglu_quantize(np.full(32, a.value, np.float32) * (np.arange(32) == 0), np.full(32, b.value, np.float32) * (np.arange(32) == 0), orc.EXP_DECLARED)[4]
                assert ok == 1 and bits(h)[0] == bits(hh)[0]
            else:
                assert ok == 0


# ---------------------------------------------------------------- committed reference-generated vectors
def test_committed_reference_vectors():
    """tests/golden/ref_vectors.npz holds outputs the compiled reference produced (tests/golden/make_ref_vectors.py);
    the inputs are regenerated from their seeds here, so this runs where the reference tree is absent."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_ref_vectors", os.path.join(HERE, "golden", "make_ref_vectors.py"))
    mk = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mk)
    gold = np.load(os.path.join(HERE, "golden", "ref_vectors.npz"))
    for seed, H, I, E, T, K in mk.LAYER_CASES:
        gate, up, down, x, ids = mk.layer_case(seed, H, I, E, T, K)
        codes, deltas, sums, _ = orc.quantize_a8(x)
        r = orc.routed_experts(H, I, K, gate, up, down, orc.Q8_0, codes, deltas, sums, ids, want_intermediates=False)
        assert np.array_equal(bits(r.rawdots), gold[f"layer_{seed}_rawdots_bits"]), seed
    rng = np.random.default_rng(300)
    vals = []
    for width in mk.ROW_WIDTHS:
        w = mk.random_q4k(rng, 1, width)[0]
        x = rng.standard_normal(width).astype(np.float32)
        codes, deltas, sums, _ = orc.quantize_a8(x[None, :])
        vals.append(orc.q4k_row_a8(w, codes[0], deltas[0], sums[0]))
    assert np.array_equal(bits(np.array(vals, np.float32)), gold["q4k_rows_bits"])
    for seed, width, count, rows in mk.GEMV_CASES:
        rng = np.random.default_rng(seed)
        w = mk.random_q8_0(rng, count, width)
        x = rng.standard_normal((rows, width)).astype(np.float32)
        codes, deltas, sums, _ = orc.quantize_a8(x)
        y, _ = orc.gemv_q8_0_a8(w, codes, deltas, width, count, threads=2)
        assert np.array_equal(bits(y), gold[f"gemv_{seed}_bits"])
    for seed, H, I, E, T, K in mk.FORMAT_LAYER_CASES:                      # Q5_K gate/up + Q5_1 down whole jobs
        gate, up, down, x, ids = mk.format_layer_case(seed, H, I, E, T, K)
        codes, deltas, sums, _ = orc.quantize_a8(x)
        r = orc.routed_experts(H, I, K, gate, up, down, orc.Q5_1, codes, deltas, sums, ids, want_intermediates=False, gate_type=orc.Q5_K)
        assert np.array_equal(bits(r.rawdots), gold[f"format_layer_{seed}_rawdots_bits"]), seed
    rng = np.random.default_rng(310)
    vals = []
    for width in mk.Q6K_WIDTHS:
        w = orc.random_q6_k(rng, (1,), width)[0]
        x = (rng.standard_normal((1, width)) * 3.0).astype(np.float32)
        codes, deltas, sums, _ = orc.quantize_a8(x, tiny_rule=True)
        vals.append(orc.q6k_down_row_a8(w, codes[0], deltas[0]))
    assert np.array_equal(bits(np.array(vals, np.float32)), gold["q6k_down_rows_bits"])
    for seed, n, rows in mk.RMSNORM_CASES:
        rng = np.random.default_rng(seed)
        x = (rng.standard_normal((rows, n)) * 2.0).astype(np.float32)
        w = rng.standard_normal(n).astype(np.float32)
        assert np.array_equal(bits(orc.rmsnorm_f32(x, w, 1e-6)), gold[f"rmsnorm_{seed}_bits"])
    for case in mk.COMBINE_CASES:                                           # the bf16-steps combine, weights / base bound or not
        eo, w, base = mk.combine_case(*case)
        assert np.array_equal(bits(orc.combine(orc.COMBINE_BF16_STEPS, w, None, eo, base)), gold[f"combine_{case[0]}_bits"]), case
        assert np.array_equal(bits(orc.combine(orc.COMBINE_BF16_STEPS_ROUNDED_EO, w, None, eo, base)), gold[f"combine_{case[0]}_rounded_bits"]), case


def test_bf16_steps_combine_against_what_the_rounding_fixes():
    """Independent of the reference build: numpy's own arithmetic restates the chain for one slot and unit weights, where
    it reduces to a single rounding (acc = bf16(0 + e)); exact ties go to even; a NaN comes back with its payload; with
    weights of one and operands that are bfloat16 values whose sums stay within 8 bits the chain is exact integer addition."""
    def bf16(a):
        b = np.asarray(a, np.float32).view(np.uint32).astype(np.uint64)
        return (((b + 0x7fff + ((b >> 16) & 1)) & 0xffff0000).astype(np.uint32)).view(np.float32)
    rng = np.random.default_rng(77)
    e = rng.standard_normal((4, 1, 50)).astype(np.float32)
    assert np.array_equal(bits(orc.combine(orc.COMBINE_BF16_STEPS, None, None, e)), bits(bf16(e[:, 0])))
    ties = np.array([[[1.00390625, 1.01171875, -1.00390625, 3.0e38]]], np.float32)
    assert orc.combine(orc.COMBINE_BF16_STEPS, None, None, ties).tolist() == [[1.0, 1.015625, -1.0, float(bf16(np.float32(3.0e38)))]]
    nan = np.array([[[0]]], np.uint32); nan[0, 0, 0] = 0x7fc12345
    assert bits(orc.combine(orc.COMBINE_BF16_STEPS, None, None, nan.view(np.float32)))[0, 0] == 0x7fc12345
    small = rng.integers(-7, 8, (3, 16, 40)).astype(np.float32)               # every partial sum is an integer of <= 8 bits
    ones = np.ones((3, 16), np.float32)
    base = rng.integers(-7, 8, (3, 40)).astype(np.float32)
    assert np.array_equal(orc.combine(orc.COMBINE_BF16_STEPS, ones, None, small, base), small.sum(axis=1) + base)
    # a weight enters as bf16(e * w), not as an fma: 3 * (1 + 2^-7) = 3.0234375 is a tie and rounds to 3.03125 before it is added
    # to 256 (259.03125 -> 260 in bfloat16, whose steps are 2 there); the fma form keeps 259.0234375
    e2 = np.array([[[256.0], [3.0]]], np.float32)
    w2 = np.array([[1.0, 1.0078125]], np.float32)
    assert orc.combine(orc.COMBINE_BF16_STEPS, w2, None, e2)[0, 0] == 260.0
    assert orc.combine(orc.COMBINE_FMA_SLOT, w2, None, e2, np.zeros((1, 1), np.float32))[0, 0] == 259.0234375


def test_vector_form_of_the_q4k_row_equals_the_plain_loop():
    """orc_q4k_row_a8 takes a vector form on hosts with AVX2 + AVX-VNNI (the reference's own fast rows are of that kind,
    src/cpu/arch/avx2/routed_expert_avx2.cpp); the plain loop is the statement of src/cpu/core/routed_expert.cpp:73-108. Same
    bits on random blocks, on extreme codes and on non-finite block scales."""
    L = orc.lib()
    if not L.orc_vector_rows(1):
        pytest.skip("this host has no AVX-VNNI: only the plain loop runs")
    rng = np.random.default_rng(2024)
    try:
        for case in range(200):
            blocks = int(rng.integers(1, 9))
            row = rng.integers(0, 256, blocks * 144, dtype=np.uint8)
            if case % 3:
                row.reshape(blocks, 144)[:, 1] = (row.reshape(blocks, 144)[:, 1] & 0x83) | 0x18        # moderate |d|
                row.reshape(blocks, 144)[:, 3] = (row.reshape(blocks, 144)[:, 3] & 0x83) | 0x18
            codes = rng.integers(-127, 128, blocks * 256, dtype=np.int8)
            if case % 5 == 0:
                codes[:] = 127 if case % 10 == 0 else -127
                row.reshape(blocks, 144)[:, 16:] = 0xFF
            deltas = (rng.standard_normal(blocks * 8) * 0.05).astype(np.float32)
            sums = codes.reshape(-1, 32).astype(np.int32).sum(axis=1).astype(np.int32)
            L.orc_vector_rows(1)
            fast = orc.q4k_row_a8(row, codes, deltas, sums)
            L.orc_vector_rows(0)
            plain = orc.q4k_row_a8(row, codes, deltas, sums)
            # (a NaN's payload depends on which operand an instruction takes it from: every NaN counts as the same value)
            assert (np.isnan(fast) and np.isnan(plain)) or np.float32(fast).view(np.uint32) == np.float32(plain).view(np.uint32), case
    finally:
        L.orc_vector_rows(1)


def test_shared_gate_order_fixtures():
    """orc_shared_gate (src/hip_shared_expert_launcher.hip:624-645): what the arithmetic fixes, on inputs where a plausible mistake
    shows. (1) the halving tree pairs lane l with l + 128, then l + 64, ...: with 2^24, 1, -2^24 + ... placed on lanes 0, 128, 64, 192
    the tree gives 1, a sequential sum 2, adjacent pairs 2. (2) each step is one fma: (2^12 + 1)^2 = 2^24 + 2^13 + 1 keeps its last
    bit only inside an fma. (3) thread t owns features t, t + 256, ... in ascending order. (4) against float64 on random rows."""
    E = orc.EXP_GFX1151
    sig = lambda d: np.float32(1.0) / (np.float32(1.0) + np.float32(orc.lib().orc_expf_gfx1151(float(-d))))
    # (1) pairing
    x = np.ones((1, 256), np.float32)
    w = np.zeros(256, np.float32)
    w[0], w[128], w[64], w[192] = 2.0 ** 24, 1.0, -(2.0 ** 24), 1.0
    gate, dots = orc.shared_gate(x, w, E)
    assert dots[0] == 1.0 and bits(gate)[0] == bits(np.array([sig(1.0)], np.float32))[0]
    # (a sum of the lanes in index order gives 2 here, and so does the adjacent pairing; a second placement of the same kind:)
    w2 = np.zeros(256, np.float32)
    w2[0], w2[1], w2[128], w2[129] = 2.0 ** 24, -(2.0 ** 24), 1.0, 1.0     # tree: (2^24 + 1) + (-2^24 + 1) = 2^24 + (-2^24 + 1) = 1; lanes in index order: 0 + 1 + 1 = 2
    _, dots2 = orc.shared_gate(x, w2, E)
    assert dots2[0] == 1.0
    # (2) fma: thread 0 takes features 0 and 256
    x3 = np.zeros((1, 512), np.float32); w3 = np.zeros(512, np.float32)
    x3[0, 0], w3[0] = -1.0, 2.0 ** 24 + 2.0 ** 13
    x3[0, 256], w3[256] = 2.0 ** 12 + 1.0, 2.0 ** 12 + 1.0
    gate3, dots3 = orc.shared_gate(x3, w3, E)
    assert dots3[0] == 1.0                                                  # product then sum would give 0
    assert bits(gate3)[0] == bits(np.array([sig(1.0)], np.float32))[0] and gate3[0] != 0.5
    # (3) ascending features within a thread: 2^24 first, then 1 twice -> 2^24 (each 1 is lost); descending would give 2^24 + 2
    x4 = np.ones((1, 768), np.float32); w4 = np.zeros(768, np.float32)
    w4[5], w4[261], w4[517] = 2.0 ** 24, 1.0, 1.0
    _, dots4 = orc.shared_gate(x4, w4, E)
    assert dots4[0] == 2.0 ** 24
    # (4) random rows against float64, and the sigmoid's fixed points
    rng = np.random.default_rng(635)
    xr = rng.standard_normal((6, 2048)).astype(np.float32)
    wr = (rng.standard_normal(2048) * 0.05).astype(np.float32)
    gate5, dots5 = orc.shared_gate(xr, wr, E)
    d64 = xr.astype(np.float64) @ wr.astype(np.float64)
    assert np.allclose(dots5, d64, rtol=0, atol=2e-5) and np.allclose(gate5, 1.0 / (1.0 + np.exp(-d64)), rtol=0, atol=1e-6)
    g0, _ = orc.shared_gate(np.zeros((1, 300), np.float32), np.ones(300, np.float32), E)
    assert g0[0] == 0.5


def test_shared_slot_enters_the_combine_as_product_then_sum():
    """orc_combine_shared: the routed slots by fma, an always-on slot as acc + (w * value). With weight 1 it is the plain combine
    (fma(1, v, acc) = acc + v); with a gate the product is rounded on its own, which a cancellation makes visible."""
    rng = np.random.default_rng(56)
    raw = rng.standard_normal((4, 5, 40)).astype(np.float32)
    w = rng.random((4, 5)).astype(np.float32)
    ids = np.tile(np.arange(5, dtype=np.uint32), (4, 1))
    base = rng.standard_normal((4, 40)).astype(np.float32)
    w1 = w.copy(); w1[:, 4] = 1.0
    assert np.array_equal(bits(orc.combine_shared(0, w1, ids, raw, 1, base)), bits(orc.combine(0, w1, ids, raw, base)))
    got = orc.combine_shared(0, w, ids, raw, 1, base)
    routed = orc.combine(0, w[:, :4].copy(), ids[:, :4].copy(), raw[:, :4].copy())
    want = (routed + (w[:, 4:5] * raw[:, 4]).astype(np.float32)).astype(np.float32) + base
    assert np.array_equal(bits(got), bits(want))
    # (1 + 2^-12)^2 = 1 + 2^-11 + 2^-24: rounded on its own the last term is lost, inside an fma it survives the cancellation
    one = np.array([[[-(1.0 + 2.0 ** -11)], [1.0 + 2.0 ** -12]]], np.float32)
    ww = np.array([[1.0, 1.0 + 2.0 ** -12]], np.float32)
    i2 = np.array([[0, 1]], np.uint32)
    assert orc.combine_shared(0, ww, i2, one, 1)[0, 0] == 0.0
    assert orc.combine(0, ww, i2, one, np.zeros((1, 1), np.float32))[0, 0] == 2.0 ** -24


def _q8_rows(scales_bits, codes):
    """Q8_0 rows from fp16 scale bit patterns [rows][blocks] and codes [rows][blocks][32]."""
    rows, blocks = scales_bits.shape
    w = np.zeros((rows, blocks, 34), np.uint8)
    w[:, :, 0], w[:, :, 1] = scales_bits & 0xff, scales_bits >> 8
    w[:, :, 2:] = codes.astype(np.int8).view(np.uint8)
    return w.reshape(rows, blocks * 34)


def test_dense_a8_profile_order_fixtures():
    """The row contract of the reference's dense A8 profile (src/hip_q8_rows_gemv.hpp:1155-1170; host statement
    tests/dense_a8_small_reference_tests.cpp:93-104) as what the arithmetic fixes: (1) one ascending chain, not the 32-lane tree of
    the CPU kernel table; (2) each step one fma; (3) the scale is float(d_w) * delta, formed first; (4) NaN scales and NaN deltas
    give the canonical NaN, an infinite scale times a zero dot as well; (5) the quantiser's rules; (6) against float64."""
    one, zero = 0x3c00, 0x0000
    # (1) blocks 0..63 with dots 2^24, 1, 1, ..., -2^24 at the end: ascending fma chain keeps 2^24 through the ones (each lost), ends at 0;
    #     lane-strided partial sums + tree (orc.gemv_q8_0_a8) give 61
    blocks = 64
    codes_x = np.zeros((1, blocks * 32), np.int8); codes_x[0, ::32] = 1                # one live code per block
    deltas = np.ones((1, blocks), np.float32)
    wcodes = np.zeros((1, blocks, 32), np.int32); wcodes[0, :, 0] = 1
    sb = np.full((1, blocks), one, np.uint16)
    deltas[0, 0], deltas[0, blocks - 1] = 2.0 ** 24, -(2.0 ** 24)
    w = _q8_rows(sb, wcodes)
    assert orc.gemv_q8_0_a8_chain(w, codes_x, deltas, blocks * 32, 1)[0, 0] == 0.0
    assert orc.gemv_q8_0_a8(w, codes_x, deltas, blocks * 32, 1)[0][0, 0] == 61.0
    # (2) fma: acc = -(2^24 + 2^13) from block 0, block 1 scale 2^12 + 1 (as delta), dot 2^12 + 1 -> exact product 2^24 + 2^13 + 1
    cx = np.zeros((1, 64), np.int8); cx[0, 0] = 1
    wc = np.zeros((1, 2, 32), np.int32); wc[0, 0, 0] = -1                              # block 0: dot -1
    wc[0, 1, 0] = wc[0, 1, 1] = 127; cx[0, 32] = cx[0, 33] = 16                        # block 1: 2 * 127 * 16 = 4064
    wc[0, 1, 2] = 33; cx[0, 34] = 1                                                    # + 33 = 4097 = 2^12 + 1
    d2 = np.array([[2.0 ** 24 + 2.0 ** 13, 2.0 ** 12 + 1.0]], np.float32)
    w2 = _q8_rows(np.full((1, 2), one, np.uint16), wc)
    assert orc.gemv_q8_0_a8_chain(w2, cx, d2, 64, 1)[0, 0] == 1.0                      # product then sum would give 0
    # (3) the three-factor product: float(d_w) * delta is rounded first, then multiplies the dot inside the fma. d_w = 1 + 2^-10,
    #     delta = 1 + 342 * 2^-23, dot = 3: the other two associations (one rounding of the whole product; d * (delta * dot)) differ
    sb3 = np.array([[0x3c01]], np.uint16)
    wc3 = np.zeros((1, 1, 32), np.int32); wc3[0, 0, 0] = 3
    cx3 = np.zeros((1, 32), np.int8); cx3[0, 0] = 1
    d3 = np.array([[1.0 + 342 * 2.0 ** -23]], np.float32)
    got = orc.gemv_q8_0_a8_chain(_q8_rows(sb3, wc3), cx3, d3, 32, 1)[0, 0]
    dw, dl = np.float32(1.0 + 2.0 ** -10), d3[0, 0]
    assert got == np.float32(np.float64(np.float32(dw * dl)) * 3.0)
    assert got != np.float32(np.float64(dw) * np.float64(dl) * 3.0) and got != np.float32(np.float64(dw) * np.float64(np.float32(dl * np.float32(3.0))))
    # (4) NaN and infinity: the reference's own scale patterns (tests/dense_a8_small_reference_tests.cpp:43-44)
    for bits_, want_nan in ((0x7e01, True), (0x7c00, True), (0xfc00, True), (0x7bff, False)):
        sbn = np.array([[bits_, one]], np.uint16)
        wcn = np.zeros((1, 2, 32), np.int32); wcn[0, 1, 0] = 5                          # block 0: dot 0 (inf * 0 = NaN), block 1: 5
        cxn = np.zeros((1, 64), np.int8); cxn[0, 32] = 1
        y = orc.gemv_q8_0_a8_chain(_q8_rows(sbn, wcn), cxn, np.ones((1, 2), np.float32), 64, 1)
        assert (bits(y)[0, 0] == 0x7fc00000) == want_nan and (want_nan or y[0, 0] == 5.0)
    nan_delta = np.array([[np.nan, 1.0]], np.float32); nan_delta.view(np.uint32)[0, 0] = 0xffc12345
    y = orc.gemv_q8_0_a8_chain(_q8_rows(np.full((1, 2), one, np.uint16), wcn), cxn, nan_delta, 64, 1)
    assert bits(y)[0, 0] == 0x7fc00000
    # (5) the quantiser
    x = np.zeros((1, 128), np.float32)
    x[0, :32] = np.linspace(-3.0, 3.0, 32)
    x[0, 40] = np.inf                                                                   # block 1: non-finite
    x[0, 64:96] = 2.0 ** -120                                                           # block 2: tiny
    c, d = orc.dense_a8_quantize(x)
    c_ref, d_ref, _, _ = orc.quantize_a8(x[:, :32].copy(), tiny_rule=True)
    assert np.array_equal(c[0, :32], c_ref[0]) and d[0, 0] == d_ref[0, 0] == np.float32(3.0) / np.float32(127.0)
    assert bits(d)[0, 1] == 0x7fc00000 and not c[0, 32:64].any()
    assert d[0, 2] == 1.0 and not c[0, 64:96].any() and d[0, 3] == 1.0 and not c[0, 96:].any()
    # (6) random rows against float64
    rng = np.random.default_rng(1155)
    wq = orc.quantize_rows(orc.Q8_0, (rng.standard_normal((24, 1024)) * 0.05).astype(np.float32))
    xr = rng.standard_normal((3, 1024)).astype(np.float32)
    cq, dq = orc.dense_a8_quantize(xr)
    cq2, dq2, _, _ = orc.quantize_a8(xr, tiny_rule=True)
    assert np.array_equal(cq, cq2) and np.array_equal(bits(dq), bits(dq2))              # finite rows: the kernel table's quantiser
    y = orc.gemv_q8_0_a8_chain(wq, cq, dq, 1024, 24)
    wd = orc.dequant_rows(orc.Q8_0, wq, 1024).astype(np.float64)
    xd = (cq.astype(np.float64).reshape(3, 32, 32) * dq.astype(np.float64)[:, :, None]).reshape(3, 1024)
    assert np.allclose(y, xd @ wd.T, rtol=0, atol=2e-5 * np.abs(xd @ wd.T).max())
