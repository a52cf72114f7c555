"""ctypes view of the parity oracle (oracle/liboracle.so) and, when it was built, of the compiled reference
(oracle/_ref/libstrix_ref.so). Test infrastructure only: the GPU library never imports this module."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")

Q5_1, Q8_0, Q4_K, Q5_K, Q6_K = 7, 8, 12, 13, 14
Q5_1_BLOCK, Q8_0_BLOCK, Q4_K_BLOCK, Q5_K_BLOCK, Q6_K_BLOCK = 24, 34, 144, 176, 210
EXP_GFX1151, EXP_DECLARED, EXP_LIBM = 0, 1, 2
LOGITS_FMA, LOGITS_LANE32 = 0, 1
COMBINE_FMA_SLOT, COMBINE_MULADD_ASC, COMBINE_BF16_STEPS, COMBINE_BF16_STEPS_ROUNDED_EO = 0, 1, 3, 4

u8p, i8p, f32p, i32p, u32p = (C.POINTER(t) for t in (C.c_uint8, C.c_int8, C.c_float, C.c_int32, C.c_uint32))


def _ptr(a, t):
    if a is None:
        return C.cast(None, t)
    assert a.flags["C_CONTIGUOUS"], "oracle arguments must be contiguous"
    return a.ctypes.data_as(t)


def build_oracle():
    """Compile the oracle (and the reference shim when /root/reference exists). Idempotent."""
    subprocess.run(["make", "-C", ORACLE_DIR, "-j8"], check=True, stdout=subprocess.DEVNULL)


def _load(path):
    return C.CDLL(path) if os.path.exists(path) else None


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        path = os.path.join(ORACLE_DIR, "liboracle.so")
        if not os.path.exists(path):
            build_oracle()
        _lib = C.CDLL(path)
        _declare(_lib)
    return _lib


def ref():
    """The compiled reference, or None when oracle/_ref was not built (no reference tree at build time)."""
    global _ref
    if _ref is None:
        _ref = _load(os.path.join(ORACLE_DIR, "_ref", "libstrix_ref.so")) or False
        if _ref:
            _ref.ref_half_to_float.restype = C.c_float
            _ref.ref_contract_half_to_float.restype = C.c_float
            _ref.ref_ggml_fp16.restype = C.c_float
            _ref.ref_declared_exp.restype = C.c_float
            _ref.ref_declared_exp.argtypes = [C.c_float]
            _ref.ref_gfx1151_expf_empty_tables.restype = C.c_float
            _ref.ref_gfx1151_expf_empty_tables.argtypes = [C.c_float]
            _ref.ref_last_error.restype = C.c_char_p
            _ref.ref_executor_create.restype = C.c_void_p
            _ref.ref_executor_isa.restype = C.c_char_p
            _ref.ref_executor_isa.argtypes = [C.c_void_p]
            _ref.ref_executor_destroy.argtypes = [C.c_void_p]
    return _ref or None


class Q8a8View(C.Structure):
    _fields_ = [("weight", C.c_void_p), ("codes", C.c_void_p), ("deltas", C.c_void_p), ("out", C.c_void_p),
                ("row_bytes", C.c_uint32), ("in_", C.c_uint32), ("count", C.c_uint32), ("rows", C.c_uint32),
                ("x_stride", C.c_uint32), ("out_stride", C.c_uint32), ("accumulate", C.c_uint32)]


class RoutePolicy(C.Structure):
    _fields_ = [("experts", C.c_uint32), ("top_k", C.c_uint32), ("logits_order", C.c_int), ("exp_kind", C.c_int),
                ("renorm_eps", C.c_float), ("scale", C.c_float), ("renormalize", C.c_int), ("renorm_single", C.c_int)]


class ExpertWeights(C.Structure):
    _fields_ = [("hidden", C.c_uint32), ("ffn", C.c_uint32), ("experts", C.c_uint32), ("top_k", C.c_uint32),
                ("gate_type", C.c_uint32), ("down_type", C.c_uint32),
                ("gate", C.c_void_p), ("up", C.c_void_p), ("down", C.c_void_p),
                ("gate_expert_stride", C.c_uint64), ("gate_row_stride", C.c_uint64),
                ("down_expert_stride", C.c_uint64), ("down_row_stride", C.c_uint64), ("exp_kind", C.c_int),
                ("swiglu_limit", C.c_float)]


class ExpertJob(C.Structure):
    _fields_ = [("codes", C.c_void_p), ("deltas", C.c_void_p), ("sums", C.c_void_p), ("ids", C.c_void_p),
                ("rows", C.c_uint32),
                ("gate_out", C.c_void_p), ("up_out", C.c_void_p), ("h_out", C.c_void_p), ("h_codes", C.c_void_p),
                ("h_deltas", C.c_void_p), ("h_sums", C.c_void_p), ("rawdots", C.c_void_p), ("status", C.c_void_p)]


def _declare(L):
    L.orc_half_to_float.restype = C.c_float
    L.orc_half_to_float.argtypes = [C.c_uint16]
    L.orc_float_to_half.restype = C.c_uint16
    L.orc_float_to_half.argtypes = [C.c_float]
    L.orc_q4k_factor_words.restype = C.c_uint
    L.orc_q4k_row_a8.restype = C.c_float
    L.orc_q5k_row_a8.restype = C.c_float
    L.orc_q6k_down_row_a8.restype = C.c_float
    L.orc_q4k_row_a8_contract_form.restype = C.c_float
    L.orc_q8_0_down_row_a8.restype = C.c_float
    L.orc_q5_1_down_row_a8.restype = C.c_float
    L.orc_expf_gfx1151.restype = C.c_float
    L.orc_expf_gfx1151.argtypes = [C.c_float]
    L.orc_declared_exp.restype = C.c_float
    L.orc_declared_exp.argtypes = [C.c_float]
    L.orc_lane_dot.restype = C.c_float
    L.orc_lane_dot.argtypes = [f32p, f32p, C.c_size_t]


# ---------------------------------------------------------------- numpy-level helpers
def rmsnorm_f32(x, w=None, eps=1e-6):
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty_like(x)
    wp = None if w is None else _ptr(np.ascontiguousarray(w, np.float32), f32p)
    lib().orc_rmsnorm_f32(_ptr(x, f32p), wp, C.c_uint32(x.shape[1]), C.c_float(eps), _ptr(y, f32p), C.c_uint32(x.shape[0]))
    return y


def row_bytes(qtype, elements):
    if qtype == Q5_1:
        return elements // 32 * Q5_1_BLOCK
    if qtype == Q5_K:
        return elements // 256 * Q5_K_BLOCK
    if qtype == Q6_K:
        return elements // 256 * Q6_K_BLOCK
    return elements // 32 * Q8_0_BLOCK if qtype == Q8_0 else elements // 256 * Q4_K_BLOCK


def half_to_float(bits):
    return lib().orc_half_to_float(int(bits))


def float_to_half(value):
    return lib().orc_float_to_half(float(np.float32(value)))


def dequant_rows(qtype, packed, elements):
    """packed: uint8 [rows][row_bytes] -> float32 [rows][elements]."""
    if qtype == Q5_K:
        return dequant_q5_k_rows(packed, elements)
    if qtype == Q5_1:
        return dequant_q5_1_rows(packed, elements)
    if qtype == Q6_K:
        return dequant_q6_k_rows(packed, elements)
    packed = np.ascontiguousarray(packed, dtype=np.uint8).reshape(-1, row_bytes(qtype, elements))
    out = np.empty((packed.shape[0], elements), np.float32)
    fn = lib().orc_dequant_q8_0_row if qtype == Q8_0 else lib().orc_dequant_q4_k_row
    for r in range(packed.shape[0]):
        fn(_ptr(packed[r], u8p), C.c_size_t(elements), _ptr(out[r], f32p))
    return out


def quantize_rows(qtype, x):
    """x: float32 [rows][elements] -> uint8 [rows][row_bytes] with the oracle's writer."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    x2 = x.reshape(-1, x.shape[-1])
    out = np.empty((x2.shape[0], row_bytes(qtype, x2.shape[1])), np.uint8)
    fn = lib().orc_quantize_q8_0_row if qtype == Q8_0 else lib().orc_quantize_q4_k_row
    for r in range(x2.shape[0]):
        fn(_ptr(x2[r], f32p), C.c_size_t(x2.shape[1]), _ptr(out[r], u8p))
    return out.reshape(x.shape[:-1] + (out.shape[1],))


def quantize_a8(x, tiny_rule=True):
    """x float32 [rows][width] -> (codes int8, deltas f32, sums i32, rc list)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    x2 = x.reshape(-1, x.shape[-1])
    rows, width = x2.shape
    codes = np.zeros((rows, width), np.int8)
    deltas = np.zeros((rows, width // 32), np.float32)
    sums = np.zeros((rows, width // 32), np.int32)
    rcs = [lib().orc_quantize_a8(_ptr(x2[r], f32p), C.c_size_t(width), _ptr(codes[r], i8p), _ptr(deltas[r], f32p),
                                 _ptr(sums[r], i32p), int(tiny_rule)) for r in range(rows)]
    return codes, deltas, sums, rcs


def gemv_q8_0_a8(weight, codes, deltas, n_in, count, out=None, accumulate=False, threads=1):
    weight = np.ascontiguousarray(weight, np.uint8)
    rows = codes.shape[0]
    if out is None:
        out = np.zeros((rows, count), np.float32)
    v = Q8a8View(weight.ctypes.data, codes.ctypes.data, deltas.ctypes.data, out.ctypes.data,
                 n_in // 32 * Q8_0_BLOCK, n_in, count, rows, codes.shape[1], out.shape[1], int(accumulate))
    rc = lib().orc_gemv_q8_0_a8(C.byref(v), threads)
    return out, rc


def q4k_row_a8(wrow, codes, deltas, sums, contract_form=False):
    wrow = np.ascontiguousarray(wrow, np.uint8)
    fn = lib().orc_q4k_row_a8_contract_form if contract_form else lib().orc_q4k_row_a8
    return np.float32(fn(_ptr(wrow, u8p), C.c_uint32(wrow.size // Q4_K_BLOCK), _ptr(codes, i8p), _ptr(deltas, f32p),
                         _ptr(sums, i32p)))


def q8_0_down_row_a8(wrow, codes, deltas):
    wrow = np.ascontiguousarray(wrow, np.uint8)
    return np.float32(lib().orc_q8_0_down_row_a8(_ptr(wrow, u8p), C.c_uint32(wrow.size // Q8_0_BLOCK), _ptr(codes, i8p),
                                                 _ptr(deltas, f32p)))


def q5_1_down_row_a8(wrow, codes, deltas, sums):
    wrow = np.ascontiguousarray(wrow, np.uint8)
    return np.float32(lib().orc_q5_1_down_row_a8(_ptr(wrow, u8p), C.c_uint32(wrow.size // Q5_1_BLOCK), _ptr(codes, i8p),
                                                 _ptr(deltas, f32p), _ptr(sums, i32p)))


def q5k_row_a8(wrow, codes, deltas, sums):
    wrow = np.ascontiguousarray(wrow, np.uint8)
    return np.float32(lib().orc_q5k_row_a8(_ptr(wrow, u8p), C.c_uint32(wrow.size // Q5_K_BLOCK), _ptr(codes, i8p), _ptr(deltas, f32p),
                                           _ptr(sums, i32p)))


def quantize_q5_k_rows(x):
    """A plain min / max Q5_K writer for tests (the reference has none): float32 [..., width] -> uint8 [..., width / 256 * 176].
    Per sub-block scale = (max - min0) / 31 and offset = -min0 (min0 = min(min, 0)), d = max scale / 63, dmin = max offset / 63
    as fp16, 6-bit factors and 5-bit codes by round-to-nearest against the fp16 values; packed as the decoders expect."""
    x = np.ascontiguousarray(x, np.float32)
    lead, width = x.shape[:-1], x.shape[-1]
    v = x.reshape(-1, width // 256, 8, 32).astype(np.float64)
    mn = np.minimum(v.min(-1), 0.0)
    scale = (v.max(-1) - mn) / 31.0
    d = (scale.max(-1) / 63.0).astype(np.float16)
    dm = ((-mn).max(-1) / 63.0).astype(np.float16)
    d64, dm64 = d.astype(np.float64), dm.astype(np.float64)
    sc = np.where(d64[..., None] > 0, np.rint(scale / np.where(d64 > 0, d64, 1.0)[..., None]), 0).clip(0, 63).astype(np.uint32)
    m = np.where(dm64[..., None] > 0, np.rint(-mn / np.where(dm64 > 0, dm64, 1.0)[..., None]), 0).clip(0, 63).astype(np.uint32)
    step = d64[..., None] * sc
    q = np.where(step[..., None] > 0, np.rint((v + (dm64[..., None] * m)[..., None]) / np.where(step > 0, step, 1.0)[..., None]), 0).clip(0, 31).astype(np.uint32)
    out = np.zeros(v.shape[:2] + (Q5_K_BLOCK,), np.uint8)
    out[..., 0:2] = d.view(np.uint8).reshape(d.shape + (2,))
    out[..., 2:4] = dm.view(np.uint8).reshape(dm.shape + (2,))
    for j in range(4):
        out[..., 4 + j] = (sc[..., j] & 63) | ((sc[..., j + 4] >> 4) << 6)
        out[..., 8 + j] = (m[..., j] & 63) | ((m[..., j + 4] >> 4) << 6)
        out[..., 12 + j] = (sc[..., j + 4] & 15) | ((m[..., j + 4] & 15) << 4)
    fifth = np.zeros(v.shape[:2] + (32,), np.uint32)
    for j in range(8):
        fifth |= (q[..., j, :] >> 4) << j
    out[..., 16:48] = fifth.astype(np.uint8)
    for p in range(4):
        out[..., 48 + 32 * p: 80 + 32 * p] = ((q[..., 2 * p, :] & 15) | ((q[..., 2 * p + 1, :] & 15) << 4)).astype(np.uint8)
    return out.reshape(lead + (width // 256 * Q5_K_BLOCK,))


def random_q5_k(rng, shape_rows, width):
    """Q5_K rows of random bytes (factors, fifth bits, nibbles) with positive fp16 d and dmin around 2^-11."""
    w = rng.integers(0, 256, tuple(shape_rows) + (width // 256 * Q5_K_BLOCK,), dtype=np.uint8)
    w[..., 1::Q5_K_BLOCK] = (w[..., 1::Q5_K_BLOCK] & 0x03) | 0x10
    w[..., 3::Q5_K_BLOCK] = (w[..., 3::Q5_K_BLOCK] & 0x03) | 0x10
    return w


def dequant_q5_k_rows(raw, width):
    """ggml Q5_K: x = d * sc_j * q - dmin * m_j, q = nibble | fifth bit << 4 (layout of src/cpu/core/routed_expert.cpp:73-108;
    factors as in Q4_K, src/cpu/core/routed_expert.cpp:65-71)."""
    raw = np.ascontiguousarray(raw, np.uint8).reshape(-1, width // 256, Q5_K_BLOCK)
    d = raw[..., 0:2].copy().view(np.float16).astype(np.float32)[..., 0]
    dm = raw[..., 2:4].copy().view(np.float16).astype(np.float32)[..., 0]
    sc_bytes = raw[..., 4:16].astype(np.uint32)
    out = np.zeros(raw.shape[:2] + (256,), np.float32)
    for j in range(8):
        if j < 4:
            sc, mn = sc_bytes[..., j] & 63, sc_bytes[..., 4 + j] & 63
        else:
            sc = (sc_bytes[..., 4 + j] & 15) | ((sc_bytes[..., j - 4] >> 6) << 4)
            mn = (sc_bytes[..., 4 + j] >> 4) | ((sc_bytes[..., j] >> 6) << 4)
        byte = raw[..., 48 + 32 * (j // 2): 48 + 32 * (j // 2) + 32].astype(np.uint32)
        q = ((byte >> 4) if j & 1 else (byte & 15)) | (((raw[..., 16:48].astype(np.uint32) >> j) & 1) << 4)
        out[..., 32 * j: 32 * j + 32] = (d * sc.astype(np.float32))[..., None] * q.astype(np.float32) - (dm * mn.astype(np.float32))[..., None]
    return out.reshape(raw.shape[0], width)


def q6k_down_row_a8(wrow, codes, deltas):
    wrow = np.ascontiguousarray(wrow, np.uint8)
    return np.float32(lib().orc_q6k_down_row_a8(_ptr(wrow, u8p), C.c_uint32(wrow.size // Q6_K_BLOCK), _ptr(codes, i8p), _ptr(deltas, f32p)))


def random_q6_k(rng, shape_rows, width):
    """Q6_K rows of random bytes (nibbles, bit pairs, signed scales) with fp16 d of either sign around 2^-13."""
    w = rng.integers(0, 256, tuple(shape_rows) + (width // 256 * Q6_K_BLOCK,), dtype=np.uint8)
    w[..., 209::Q6_K_BLOCK] = (w[..., 209::Q6_K_BLOCK] & 0x83) | 0x08
    return w


def dequant_q6_k_rows(raw, width):
    """ggml dequantize_row_q6_K: x = d * scale[16-weight group] * (q - 32), element layout of src/moe_a8_down_contract.cpp:20-29."""
    raw = np.ascontiguousarray(raw, np.uint8).reshape(-1, width // 256, Q6_K_BLOCK)
    d = raw[..., 208:210].copy().view(np.float16).astype(np.float32)[..., 0]
    scales = raw[..., 192:208].view(np.int8).astype(np.float32)
    out = np.zeros(raw.shape[:2] + (256,), np.float32)
    for j in range(8):
        half, quarter = j // 4, j % 4
        ql = raw[..., half * 64 + (quarter & 1) * 32: half * 64 + (quarter & 1) * 32 + 32].astype(np.int32)
        qh = raw[..., 128 + half * 32: 128 + half * 32 + 32].astype(np.int32)
        q = (((ql >> (4 if quarter >= 2 else 0)) & 15) | (((qh >> (2 * quarter)) & 3) << 4)) - 32
        sc = np.repeat(scales[..., 2 * j: 2 * j + 2], 16, axis=-1)
        out[..., 32 * j: 32 * j + 32] = d[..., None] * sc * q.astype(np.float32)
    return out.reshape(raw.shape[0], width)


def random_q5_1(rng, shape_rows, width):
    """Q5_1 rows of random bytes (every nibble and fifth bit) with finite fp16 d and m of either sign around 2^-6."""
    w = rng.integers(0, 256, tuple(shape_rows) + (width // 32 * Q5_1_BLOCK,), dtype=np.uint8)
    w[..., 1::Q5_1_BLOCK] = (w[..., 1::Q5_1_BLOCK] & 0x83) | 0x20
    w[..., 3::Q5_1_BLOCK] = (w[..., 3::Q5_1_BLOCK] & 0x83) | 0x20
    return w


def dequant_q5_1_rows(raw, width):
    """ggml Q5_1: x_k = d * q_k + m, q_k = nibble | fifth bit << 4 (the layout of src/cpu/core/routed_expert.cpp:121-131)."""
    raw = np.ascontiguousarray(raw, np.uint8).reshape(-1, width // 32, Q5_1_BLOCK)
    d = raw[..., 0:2].copy().view(np.float16).astype(np.float32)
    m = raw[..., 2:4].copy().view(np.float16).astype(np.float32)
    fifth = raw[..., 4:8].copy().view(np.uint32)
    nib = raw[..., 8:24]
    k = np.arange(32)
    q = np.where(k < 16, nib[..., k % 16] & 15, nib[..., k % 16] >> 4).astype(np.uint32) | (((fifth >> k) & 1) << 4)
    return (d * q.astype(np.float32) + m).reshape(raw.shape[0], width)


def swiglu_quantize(g, u, exp_kind=EXP_GFX1151, limit=float("inf")):
    g = np.ascontiguousarray(g, np.float32)
    u = np.ascontiguousarray(u, np.float32)
    codes = np.zeros(32, np.int8)
    delta = C.c_float(0)
    s = C.c_int32(0)
    h = np.zeros(32, np.float32)
    ok = lib().orc_swiglu_quantize_clamped(exp_kind, C.c_float(limit), _ptr(g, f32p), _ptr(u, f32p), _ptr(codes, i8p), C.byref(delta),
                                           C.byref(s), _ptr(h, f32p))
    return ok, codes, np.float32(delta.value), s.value, h


def route(x, w, top_k, bias=None, logits_order=LOGITS_FMA, exp_kind=EXP_DECLARED, renorm_eps=0.0, scale=1.0,
          renormalize=True, threads=0, renorm_single=True):
    x = np.ascontiguousarray(x, np.float32)
    w = np.ascontiguousarray(w, np.float32)
    rows, hidden = x.shape
    experts = w.shape[0]
    p = RoutePolicy(experts, top_k, logits_order, exp_kind, renorm_eps, scale, int(renormalize), int(renorm_single))
    ids = np.zeros((rows, top_k), np.uint32)
    weights = np.zeros((rows, top_k), np.float32)
    scores = np.zeros((rows, experts), np.float32)
    logits = np.zeros((rows, experts), np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, np.float32)
    lib().orc_route(C.byref(p), _ptr(x, f32p), rows, hidden, _ptr(w, f32p), _ptr(b, f32p), _ptr(ids, u32p),
                    _ptr(weights, f32p), _ptr(scores, f32p), _ptr(logits, f32p), threads or lib().orc_max_threads())
    return ids, weights, scores, logits


def route_select(scores, top_k, renorm_eps=0.0, scale=1.0, renormalize=True, renorm_single=True):
    scores = np.ascontiguousarray(scores, np.float32)
    p = RoutePolicy(scores.size, top_k, 0, 0, renorm_eps, scale, int(renormalize), int(renorm_single))
    ids = np.zeros(top_k, np.uint32)
    weights = np.zeros(top_k, np.float32)
    lib().orc_route_select(C.byref(p), _ptr(scores, f32p), _ptr(ids, u32p), _ptr(weights, f32p))
    return ids, weights


def combine(form, w, ids, raw, base=None):
    rows, top_k, width = raw.shape
    raw = np.ascontiguousarray(raw, np.float32)
    w = None if w is None else np.ascontiguousarray(w, np.float32)
    ids = np.zeros((rows, top_k), np.uint32) if ids is None else np.ascontiguousarray(ids, np.uint32)
    y = np.zeros((rows, width), np.float32)
    b = None if base is None else np.ascontiguousarray(base, np.float32)
    lib().orc_combine(form, rows, top_k, width, _ptr(w, f32p), _ptr(ids, u32p), _ptr(raw, f32p), _ptr(b, f32p), _ptr(y, f32p))
    return y


def combine_shared(form, w, ids, raw, shared_slots, base=None):
    rows, top_k, width = raw.shape
    raw, w, ids = np.ascontiguousarray(raw, np.float32), np.ascontiguousarray(w, np.float32), np.ascontiguousarray(ids, np.uint32)
    y = np.zeros((rows, width), np.float32)
    b = None if base is None else np.ascontiguousarray(base, np.float32)
    lib().orc_combine_shared(form, rows, top_k, shared_slots, width, _ptr(w, f32p), _ptr(ids, u32p), _ptr(raw, f32p), _ptr(b, f32p), _ptr(y, f32p))
    return y


def dense_a8_quantize(x):
    x = np.ascontiguousarray(x, np.float32)
    rows, width = x.shape
    codes, deltas = np.zeros((rows, width), np.int8), np.zeros((rows, width // 32), np.float32)
    for r in range(rows):
        lib().orc_dense_a8_quantize(_ptr(x[r], f32p), width, _ptr(codes[r], i8p), _ptr(deltas[r], f32p))
    return codes, deltas


def gemv_q8_0_a8_chain(weight, codes, deltas, n_in, count):
    weight, codes, deltas = np.ascontiguousarray(weight, np.uint8), np.ascontiguousarray(codes, np.int8), np.ascontiguousarray(deltas, np.float32)
    rows = codes.shape[0]
    out = np.zeros((rows, count), np.float32)
    lib().orc_gemv_q8_0_a8_chain(_ptr(weight, u8p), n_in // 32 * 34, _ptr(codes, i8p), _ptr(deltas, f32p), n_in, count, rows, codes.shape[1], _ptr(out, f32p), count)
    return out


def shared_gate(x, w, exp_kind=EXP_GFX1151):
    x, w = np.ascontiguousarray(x, np.float32), np.ascontiguousarray(w, np.float32)
    rows, hidden = x.shape
    gate, dots = np.zeros(rows, np.float32), np.zeros(rows, np.float32)
    lib().orc_shared_gate(_ptr(x, f32p), _ptr(w, f32p), rows, hidden, exp_kind, _ptr(gate, f32p), _ptr(dots, f32p))
    return gate, dots


class ExpertResult:
    pass


def routed_experts(hidden, ffn, top_k, gate, up, down, down_type, codes, deltas, sums, ids, exp_kind=EXP_GFX1151,
                   gate_expert_stride=None, gate_row_stride=None, down_expert_stride=None, down_row_stride=None,
                   threads=0, want_intermediates=True, down_only_from=None, gate_type=Q4_K, swiglu_limit=float("inf")):
    """gate/up/down: uint8 arrays holding every expert (GGUF order unless strides are given).
    down_only_from: (h_codes, h_deltas, h_sums) -> run the down phase alone on that image."""
    gate = np.ascontiguousarray(gate, np.uint8)
    up = np.ascontiguousarray(up, np.uint8)
    down = np.ascontiguousarray(down, np.uint8)
    rows = codes.shape[0]
    grb = gate_row_stride or row_bytes(gate_type, hidden)
    geb = gate_expert_stride or grb * ffn
    drb = down_row_stride or row_bytes(down_type, ffn)
    deb = down_expert_stride or drb * hidden
    w = ExpertWeights(hidden, ffn, 0, top_k, gate_type, down_type, gate.ctypes.data, up.ctypes.data, down.ctypes.data,
                      geb, grb, deb, drb, exp_kind, swiglu_limit)
    ids = np.ascontiguousarray(ids, np.uint32)
    n = rows * top_k
    r = ExpertResult()
    r.rawdots = np.zeros((rows, top_k, hidden), np.float32)
    r.status = np.zeros(rows, np.uint32)
    if down_only_from is not None:
        r.h_codes, r.h_deltas, r.h_sums = (np.ascontiguousarray(a) for a in down_only_from)
        r.gate = r.up = r.h = None
    else:
        r.h_codes = np.zeros((n, ffn), np.int8)
        r.h_deltas = np.zeros((n, ffn // 32), np.float32)
        r.h_sums = np.zeros((n, ffn // 32), np.int32)
        r.gate = np.zeros((n, ffn), np.float32) if want_intermediates else None
        r.up = np.zeros((n, ffn), np.float32) if want_intermediates else None
        r.h = np.zeros((n, ffn), np.float32) if want_intermediates else None
    job = ExpertJob(codes.ctypes.data, deltas.ctypes.data, sums.ctypes.data, ids.ctypes.data, rows,
                    r.gate.ctypes.data if r.gate is not None else None, r.up.ctypes.data if r.up is not None else None,
                    r.h.ctypes.data if r.h is not None else None, r.h_codes.ctypes.data, r.h_deltas.ctypes.data,
                    r.h_sums.ctypes.data, r.rawdots.ctypes.data, r.status.ctypes.data)
    t = threads or lib().orc_max_threads()
    if down_only_from is not None:
        lib().orc_routed_down(C.byref(w), C.byref(job), t)
        r.bad = 0
    else:
        r.bad = lib().orc_routed_experts(C.byref(w), C.byref(job), t)
    return r


def base_linear(qtype, weight, row_stride, outputs, n_in, x, threads=0):
    weight = np.ascontiguousarray(weight, np.uint8)
    x = np.ascontiguousarray(x, np.float32)
    rows = x.shape[0]
    y = np.zeros((rows, outputs), np.float32)
    lib().orc_base_linear(qtype, _ptr(weight, u8p), C.c_uint64(row_stride), outputs, n_in, _ptr(x, f32p), rows,
                          x.shape[1], _ptr(y, f32p), outputs, threads or lib().orc_max_threads())
    return y


# ---------------------------------------------------------------- expert union of a verify window
UNION_MAX_ROWS, UNION_MAX_TOP_K, UNION_NO_SLOT, UNION_PLAN_BYTES = 8, 16, 0xFF, 16 + 128 * 12


def expert_union_build(ids, rows, top_k, experts):
    """The host reference of the union plan (include/strix/moe/expert_union.hpp:34-57): the distinct experts of rows x top_k
    ids in first-occurrence order of (row, slot) ascending, each with the slot every row holds it in (0xff: not chosen).
    Returns [(expert, [slot of row 0..7])]. ValueError on a shape outside R <= 8, K <= 16, an id >= experts, or an id
    repeated within one row."""
    ids = [int(v) for v in np.asarray(ids).reshape(-1)]
    if not (1 <= rows <= UNION_MAX_ROWS and 1 <= top_k <= UNION_MAX_TOP_K) or len(ids) != rows * top_k:
        raise ValueError("expert union: rows <= 8, top_k <= 16 and rows x top_k ids required")
    out = []
    for r in range(rows):
        for s in range(top_k):
            e = ids[r * top_k + s]
            if e >= experts:
                raise ValueError("expert union: expert id out of range")
            u = next((i for i, entry in enumerate(out) if entry[0] == e), len(out))
            if u == len(out):
                out.append((e, [UNION_NO_SLOT] * UNION_MAX_ROWS))
            if out[u][1][r] != UNION_NO_SLOT:
                raise ValueError("expert union: expert repeated within one row")
            out[u][1][r] = s
    return out


def expert_union_plan_bytes(entries, rows, top_k):
    """The device layout of a plan (expert_union.hpp:17-27): Header {count, rows, top_k, 0}, then 128 Entry {u32 expert,
    u8 slot[8]}; the entries past count as the device builder leaves them (expert 0, 0xff slots)."""
    plan = np.zeros(UNION_PLAN_BYTES, np.uint8)
    plan[:16] = np.array([len(entries), rows, top_k, 0], np.uint32).view(np.uint8)
    body = plan[16:].reshape(128, 12)
    body[:, 4:] = UNION_NO_SLOT
    for u, (e, slots) in enumerate(entries):
        body[u, :4] = np.array([e], np.uint32).view(np.uint8)
        body[u, 4:] = np.array(slots, np.uint8)
    return plan
