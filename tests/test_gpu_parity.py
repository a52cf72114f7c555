"""GPU parity tests: every value comes through the C ABI (libmi355_strix.so) and is compared with the CPU oracle on the
same seeded inputs. Integer / byte / index results and the declared fp32 chains must be bit-exact; whole-layer outputs
are additionally held to the stated tolerances (fp32-accumulated outputs: max relative error 1e-3; fp16 activations
2e-3), with "relative" = |gpu - ref| / rms(ref) and the elementwise form restricted to |ref| > 1e-2 rms(ref)."""
import ctypes as C

import numpy as np
import pytest
import torch

import orc

pytestmark = pytest.mark.gpu
TOL_F32, TOL_F16 = 1e-3, 2e-3


# plan words: header [0, 16), ticket words [16, 272), the words of the early-routes decode layer [272, 2240), then offsets / touched /
# order / items
PLAN_OFFSETS_AT = 2240

def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def rel_err(got, want):
    want64 = want.astype(np.float64)
    rms = np.sqrt(np.mean(want64 ** 2)) + 1e-30
    abs_over_rms = np.max(np.abs(got - want64)) / rms
    big = np.abs(want64) > 1e-2 * rms
    elementwise = np.max(np.abs(got[big] - want64[big]) / np.abs(want64[big])) if big.any() else 0.0
    return abs_over_rms, elementwise


def random_q4k(rng, shape_rows, width):
    w = rng.integers(0, 256, shape_rows + (width // 256 * 144,), dtype=np.uint8)
    w[..., 1::144] = (w[..., 1::144] & 0x03) | 0x0C | (rng.integers(0, 2, w[..., 1::144].shape, dtype=np.uint8) << 4)
    w[..., 3::144] = (w[..., 3::144] & 0x03) | 0x0C
    return w


# ------------------------------------------------------------------------------------------- RMSNorm
@pytest.mark.parametrize("n,rows", [(64, 3), (511, 2), (512, 5), (2048, 8), (4096, 300), (6144, 16)])
def test_rmsnorm_bit_exact(strix, n, rows):
    """mi355_rmsnorm_f32 against the oracle (itself bitwise equal to the compiled reference kernel table): the lane-strided
    fma chains, the halving tree, the correctly rounded 1 / sqrt and the two products, bit for bit."""
    rng = np.random.default_rng(n + rows)
    x = (rng.standard_normal((rows, n)) * 3.0).astype(np.float32)
    w = rng.standard_normal(n).astype(np.float32)
    assert np.array_equal(bits(strix.rmsnorm_f32(dev(x), dev(w)).cpu().numpy()), bits(orc.rmsnorm_f32(x, w)))
    assert np.array_equal(bits(strix.rmsnorm_f32(dev(x), None, eps=1e-5).cpu().numpy()), bits(orc.rmsnorm_f32(x, None, 1e-5)))


# ------------------------------------------------------------------------------------------- block decode / writers
@pytest.mark.parametrize("qtype,width", [(orc.Q8_0, 4096), (orc.Q4_K, 2048), (orc.Q4_K, 5120)])
def test_dequantised_weights_bit_exact(strix, qtype, width):
    rng = np.random.default_rng(100 + width)
    rb = orc.row_bytes(qtype, width)
    raw = rng.integers(0, 256, (37, rb), dtype=np.uint8)
    if qtype == orc.Q8_0:   # every fp16 scale pattern incl. subnormals, infinities excluded from the bit compare below
        raw[:, 1::34] &= 0xFB
    else:
        raw[:, 1::144] &= 0xFB
        raw[:, 3::144] &= 0xFB
    got = strix.dequantize_rows(qtype, dev(raw), width).cpu().numpy()
    want = orc.dequant_rows(qtype, raw, width)
    assert np.array_equal(bits(got), bits(want))


def test_fp16_scale_decode_all_65536_values(strix):
    blocks = np.zeros((65536, 34), np.uint8)
    h = np.arange(65536, dtype=np.uint16)
    blocks[:, 0], blocks[:, 1], blocks[:, 2] = h & 255, h >> 8, 1
    got = strix.dequantize_rows(orc.Q8_0, dev(blocks.reshape(64, -1)), 1024 * 32).cpu().numpy().reshape(65536, 32)[:, 0]
    want = h.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan) and np.array_equal(bits(got)[~nan], bits(want)[~nan])


@pytest.mark.parametrize("qtype", [orc.Q8_0, orc.Q4_K])
def test_weight_writers_match_oracle_bytes(strix, qtype):
    rng = np.random.default_rng(7)
    x = (rng.standard_normal((64, 2048)) * 0.02).astype(np.float32)
    x[3, :64] = 0
    x[5, 256:512] = np.abs(x[5, 256:512])
    got = strix.quantize_weight_rows(qtype, dev(x)).cpu().numpy()
    assert np.array_equal(got, orc.quantize_rows(qtype, x))


# ------------------------------------------------------------------------------------------- A8 quantiser
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_quantize_a8_bit_exact(strix, dtype):
    rng = np.random.default_rng(11)
    x = rng.standard_normal((9, 5120)).astype(dtype)
    x[1, :32] = 0
    x[2, 32:64] = dtype(6e-8) if dtype == np.float16 else 1e-37
    x[3, 64:96] *= dtype(100)
    if dtype == np.float32:
        x[4, :32] = np.float32(2.0 ** -120)     # tiny rule: codes 0, delta 1
        x[4, 32:64] = np.float32(2.0 ** -119)   # not tiny
        x[5, 0], x[5, 1] = np.array([0x3A8BE27E, 0x37B03B95], np.uint32).view(np.float32)  # division-then-round hard case
        x[5, 2:32] = 0
    codes, deltas, sums, status = strix.quantize_a8(dev(x))
    c, d, s, _ = orc.quantize_a8(x.astype(np.float32), tiny_rule=True)
    assert np.array_equal(codes.cpu().numpy(), c)
    assert np.array_equal(bits(deltas.cpu().numpy()), bits(d))
    assert np.array_equal(sums.cpu().numpy(), s)
    assert np.all(status.cpu().numpy() == 0)


def test_quantize_a8_rejects_partial_group_before_any_write(strix):
    x = torch.ones((1, 64), device="cuda")
    codes = torch.full((1, 64), 17, dtype=torch.int8, device="cuda")
    deltas = torch.full((1, 2), 19.0, device="cuda")
    for width in (31, 33):
        rc = strix.lib().mi355_quantize_a8(C.c_void_p(x.data_ptr()), 0, 1, width, C.c_uint64(256), C.c_void_p(codes.data_ptr()),
                                           C.c_void_p(deltas.data_ptr()), None, None, None)
        assert rc == strix.E_INVALID_ARGUMENT and b"multiple of 32" in strix.lib().mi355_last_error()
    torch.cuda.synchronize()
    assert bool((codes == 17).all()) and bool((deltas == 19).all())


def test_nonfinite_activation_sets_status(strix):
    x = torch.randn((3, 256), device="cuda")
    x[1, 7] = float("inf")
    *_, status = strix.quantize_a8(x)
    assert status.cpu().tolist() == [0, strix.STATUS_NONFINITE_ACTIVATION, 0]


# ------------------------------------------------------------------------------------------- config 1: dense Q8_0 GEMV
def test_config1_dense_q8_0_gemv_bit_exact(strix):
    """BASELINE config 1: x[4096] ~ N(0,1) fp32, W 4096x4096 ~ N(0,0.02) -> Q8_0 by the ggml rule, y = W x."""
    rng = np.random.default_rng(1)
    x = rng.standard_normal((1, 4096)).astype(np.float32)
    w = orc.quantize_rows(orc.Q8_0, (rng.standard_normal((4096, 4096)) * 0.02).astype(np.float32))
    codes, deltas, _, _ = strix.quantize_a8(dev(x))
    y = strix.gemv_q8_0_a8(dev(w), codes, deltas, 4096, 4096).cpu().numpy()
    c, d, s, _ = orc.quantize_a8(x)
    want, _ = orc.gemv_q8_0_a8(w, c, d, 4096, 4096, threads=8)
    assert np.array_equal(bits(y), bits(want))
    exact = x.astype(np.float64) @ orc.dequant_rows(orc.Q8_0, w, 4096).astype(np.float64).T
    assert rel_err(y, exact.astype(np.float32))[0] < 2e-2    # informational: distance of the A8 class from exact weights


def test_q8_0_gemv_order_fixture_rows_accumulate_and_padding(strix):
    g = 33
    w = np.zeros(g * 34, np.uint8)
    w[1::34], w[2::34] = 0x3C, 1
    codes = np.ones((1, g * 32), np.int8)
    deltas = np.zeros((1, g), np.float32)
    deltas[0, 0], deltas[0, 16], deltas[0, 1], deltas[0, 32] = 2.0 ** 24, -2.0 ** 24, 1, 1
    y = torch.full((1, 1), -1.0, device="cuda")
    strix.gemv_q8_0_a8(dev(w), dev(codes), dev(deltas), g * 32, 1, out=y)
    assert y.item() == 1.0
    y.fill_(-1.0)
    strix.gemv_q8_0_a8(dev(w), dev(codes), dev(deltas), g * 32, 1, out=y, accumulate=True)
    assert y.item() == 0.0
    # 11 rows x 19 outputs with padded strides, against the oracle
    rng = np.random.default_rng(3)
    x = rng.standard_normal((11, 1024)).astype(np.float32)
    wq = orc.quantize_rows(orc.Q8_0, (rng.standard_normal((19, 1024)) * 0.02).astype(np.float32))
    c, d, s, _ = orc.quantize_a8(x)
    out = torch.full((11, 24), 29.0, device="cuda")
    strix.gemv_q8_0_a8(dev(wq), dev(c), dev(d), 1024, 19, out=out)
    want, _ = orc.gemv_q8_0_a8(wq, c, d, 1024, 19)
    got = out.cpu().numpy()
    assert np.array_equal(bits(got[:, :19]), bits(want)) and np.all(got[:, 19:] == 29.0)
    # 1, 2 and 3 rows (their own instantiations), and the same weights at a pointer that is only 2-byte aligned
    shifted = torch.zeros(wq.size + 2, dtype=torch.uint8, device="cuda")
    shifted[2:] = dev(wq).reshape(-1)
    for rows in (1, 2, 3):
        for weight in (dev(wq), shifted[2:]):
            got = strix.gemv_q8_0_a8(weight, dev(c[:rows]), dev(d[:rows]), 1024, 19).cpu().numpy()
            assert np.array_equal(bits(got), bits(want[:rows]))
    v = strix.Q8a8View(1, 1, 1, 1, 68, 33, 1, 1, 64, 1, 0)
    assert strix.lib().mi355_gemv_q8_0_a8(C.byref(v), None) == strix.E_INVALID_ARGUMENT


# ------------------------------------------------------------------------------------------- router
@pytest.mark.parametrize("experts,hidden,rows,bias", [(128, 2048, 8, False), (256, 4096, 32, True), (160, 6144, 16, False)])
def test_router_topk_ids_bit_exact(strix, experts, hidden, rows, bias):
    rng = np.random.default_rng(experts)
    x = rng.standard_normal((rows, hidden)).astype(np.float16)
    wr = (rng.standard_normal((experts, hidden)) * 0.02).astype(np.float32)
    b = (rng.standard_normal(experts) * 1.5).astype(np.float32) if bias else None
    ids, wts, scores = strix.route(dev(x), dev(wr), 8, bias=None if b is None else dev(b))
    ids_ref, w_ref, s_ref, _ = orc.route(x.astype(np.float32), wr, 8, bias=b)
    assert np.array_equal(ids.cpu().numpy().astype(np.uint32), ids_ref)
    assert np.array_equal(bits(wts.cpu().numpy()), bits(w_ref))
    assert np.array_equal(bits(scores.cpu().numpy()), bits(s_ref))


def test_router_exact_ties_lane32_order_and_policy_constants(strix):
    rng = np.random.default_rng(5)
    x = np.zeros((4, 256), np.float16)
    x[:, 0] = 1
    wr = np.zeros((64, 256), np.float32)
    wr[:, 0] = (rng.integers(-8, 9, 64) / 4.0)           # many exact ties: the lower id must win
    ids, wts, _ = strix.route(dev(x), dev(wr), 6, renorm_eps=1e-20, scale=2.5)
    ids_ref, w_ref, _, _ = orc.route(x.astype(np.float32), wr, 6, renorm_eps=1e-20, scale=2.5)
    assert np.array_equal(ids.cpu().numpy().astype(np.uint32), ids_ref) and np.array_equal(bits(wts.cpu().numpy()), bits(w_ref))
    x = rng.standard_normal((3, 512)).astype(np.float32)
    wr = (rng.standard_normal((32, 512)) * 0.05).astype(np.float32)
    ids, wts, sc = strix.route(dev(x), dev(wr), 4, logits_order=strix.LOGITS_LANE32)
    ids_ref, w_ref, s_ref, _ = orc.route(x, wr, 4, logits_order=orc.LOGITS_LANE32)
    assert np.array_equal(ids.cpu().numpy().astype(np.uint32), ids_ref) and np.array_equal(bits(sc.cpu().numpy()), bits(s_ref))


@pytest.mark.parametrize("experts,hidden,rows", [(128, 2048, 8), (256, 4096, 40)])
def test_router_with_the_c_library_exp(strix, experts, hidden, rows):
    """Math::exp = expf of the C library, the exp of the reference's router test oracle (tests/hip_moe_route_launcher_tests.hip:329):
    ids, weights and scores equal the oracle's (whose exp is the host library's expf) bit for bit, for the decode and the batch
    router and through the fused layer entry."""
    rng = np.random.default_rng(experts + 1)
    x = rng.standard_normal((rows, hidden)).astype(np.float16)
    wr = (rng.standard_normal((experts, hidden)) * 0.05).astype(np.float32)
    ids, wts, scores = strix.route(dev(x), dev(wr), 8, exp_kind=strix.EXP_LIBM)
    ids_ref, w_ref, s_ref, _ = orc.route(x.astype(np.float32), wr, 8, exp_kind=orc.EXP_LIBM)
    assert np.array_equal(bits(scores.cpu().numpy()), bits(s_ref))
    assert np.array_equal(ids.cpu().numpy().astype(np.uint32), ids_ref) and np.array_equal(bits(wts.cpu().numpy()), bits(w_ref))
    _, _, s_declared, _ = orc.route(x.astype(np.float32), wr, 8, exp_kind=orc.EXP_DECLARED)
    assert not np.array_equal(bits(s_declared), bits(s_ref))      # the policy field is not ignored


def test_router_single_expert_renormalisation(strix):
    """top_k = 1: the weight is renormalised only when the policy's renorm_single is set (include/strix/moe/route_policy.hpp:146)."""
    rng = np.random.default_rng(12)
    x = rng.standard_normal((5, 512)).astype(np.float16)
    wr = (rng.standard_normal((24, 512)) * 0.05).astype(np.float32)
    for single in (False, True):
        ids, wts, _ = strix.route(dev(x), dev(wr), 1, renorm_eps=1e-20, scale=2.5, renorm_single=single)
        ids_ref, w_ref, _, _ = orc.route(x.astype(np.float32), wr, 1, renorm_eps=1e-20, scale=2.5, renorm_single=single)
        assert np.array_equal(ids.cpu().numpy().astype(np.uint32), ids_ref) and np.array_equal(bits(wts.cpu().numpy()), bits(w_ref))
    assert float(wts[0, 0]) == 2.5


# ------------------------------------------------------------------------------------------- routed experts, stage by stage
def make_layer(rng, H, I, E, full_entropy=False):
    if full_entropy:
        return random_q4k(rng, (E, I), H), random_q4k(rng, (E, I), H), random_q4k(rng, (E, H), I)
    q = lambda shape: orc.quantize_rows(orc.Q4_K, (rng.standard_normal(shape) * 0.02).astype(np.float32))
    return q((E, I, H)), q((E, I, H)), q((E, H, I))


def run_layer_both(strix, H, I, E, K, T, seed, full_entropy=False, combine=0, exp_kind=0, tp=None):
    rng = np.random.default_rng(seed)
    gate, up, down = make_layer(rng, H, I, E, full_entropy)
    x = rng.standard_normal((T, H)).astype(np.float16)
    wr = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    ids_ref, w_ref, _, _ = orc.route(x.astype(np.float32), wr, K)
    kw, okw, ffn = {}, {}, I
    g_np, u_np, d_np = gate, up, down
    if tp is not None:   # this rank's share of every expert, read in place from the unsplit tensors through strides
        rank, ranks = tp
        ffn = I // ranks
        grb, drb = H // 256 * 144, I // 256 * 144
        kw = dict(gate_expert_stride=I * grb, gate_row_stride=grb, down_expert_stride=H * drb, down_row_stride=drb)
        okw = kw
        g_np, u_np, d_np = gate.reshape(-1)[rank * ffn * grb:], up.reshape(-1)[rank * ffn * grb:], down.reshape(-1)[rank * (ffn // 256) * 144:]
    gd, ud, dd = dev(gate.reshape(-1)), dev(up.reshape(-1)), dev(down.reshape(-1))
    if tp is not None:
        off_g, off_d = tp[0] * ffn * (H // 256 * 144), tp[0] * (ffn // 256) * 144
        gd_v, ud_v, dd_v = gd[off_g:], ud[off_g:], dd[off_d:]
    else:
        gd_v, ud_v, dd_v = gd, ud, dd
    layer = strix.MoeLayer(H, ffn, E, K, gd_v, ud_v, dd_v, T, exp_kind=exp_kind, intermediates=True, **kw)
    y = layer.run(dev(x), dev(ids_ref.astype(np.int32)), dev(w_ref), combine=combine).cpu().numpy()
    c, d, s, _ = orc.quantize_a8(x.astype(np.float32))
    ref = orc.routed_experts(H, ffn, K, g_np, u_np, d_np, orc.Q4_K, c, d, s, ids_ref, exp_kind=exp_kind, **okw)
    want = orc.combine(combine, w_ref, ids_ref, ref.rawdots)
    return layer, y, ref, want, (c, d, s), ids_ref, w_ref, (g_np, u_np, d_np, ffn, okw)


def check_layer_stages(strix, layer, y, ref, want, a8, ids_ref, w_ref, tensors, H, K, T, combine, exp_kind, tol):
    g_np, u_np, d_np, ffn, okw = tensors
    c, d, s = a8
    n = T * K
    # (1) device A8 image of the input == oracle
    assert np.array_equal(layer.codes[:T].cpu().numpy(), c) and np.array_equal(bits(layer.deltas[:T].cpu().numpy()), bits(d))
    assert np.array_equal(layer.sums[:T].cpu().numpy(), s)
    # (2) device gate / up bits == oracle (the declared fp32 chain, any lane schedule)
    assert np.array_equal(bits(layer.gate_out[:n].cpu().numpy()), bits(ref.gate))
    assert np.array_equal(bits(layer.up_out[:n].cpu().numpy()), bits(ref.up))
    # (3) the device's own h, re-quantised on the CPU, == the device's down image (so exp never enters a bit compare) ...
    h_dev = layer.h_out[:n].cpu().numpy()
    hc, hd, hs, _ = orc.quantize_a8(h_dev, tiny_rule=True)
    dc, dd_, ds = layer.down_codes[:n].cpu().numpy(), layer.down_deltas[:n].cpu().numpy(), layer.down_sums[:n].cpu().numpy()
    assert np.array_equal(dc, hc) and np.array_equal(bits(dd_), bits(hd)) and np.array_equal(ds, hs)
    # ... and h itself is within an ulp or two of the oracle's h (the device exp2 in double vs the host's)
    assert np.max(np.abs(h_dev - ref.h)) <= 4e-7 * np.max(np.abs(ref.h))
    h_codes_equal = np.array_equal(dc, ref.h_codes)
    # (4) device rawdot bits == oracle down rows evaluated on the DEVICE's down image
    ref_down = orc.routed_experts(H, ffn, K, g_np, u_np, d_np, orc.Q4_K, c, d, s, ids_ref, exp_kind=exp_kind,
                                  down_only_from=(dc, dd_, ds), **okw)
    raw_dev = layer.rawdots[:T].cpu().numpy()
    assert np.array_equal(bits(raw_dev), bits(ref_down.rawdots))
    # (5) combine bits from the device rawdots
    assert np.array_equal(bits(y), bits(orc.combine(combine, w_ref, ids_ref, raw_dev)))
    # (6) whole layer vs the oracle end to end: tolerance, and bit-exact whenever the h codes agree
    a, e = rel_err(y, want)
    assert a < tol and e < tol, (a, e)
    if h_codes_equal:
        assert np.array_equal(bits(y), bits(want))
    assert np.all(layer.status[:T].cpu().numpy() == 0)
    return h_codes_equal


@pytest.mark.parametrize("H,I,E,K,T,full", [(512, 256, 6, 2, 3, False), (2048, 768, 16, 8, 8, False), (768, 512, 5, 3, 11, True),
                                            (2560, 256, 4, 2, 1, True)])
def test_moe_layer_stage_by_stage_bit_exact(strix, H, I, E, K, T, full):
    out = run_layer_both(strix, H, I, E, K, T, seed=H + T, full_entropy=full)
    check_layer_stages(strix, *out[:7], out[7], H, K, T, 0, 0, TOL_F16)


def test_moe_layer_declared_exp_is_bit_exact_end_to_end(strix):
    """With the declared exp (basic IEEE operations only) host and device share every bit of the layer."""
    H, I, E, K, T = 1024, 512, 8, 4, 5
    layer, y, ref, want, *_ = run_layer_both(strix, H, I, E, K, T, seed=77, exp_kind=1)
    assert np.array_equal(layer.down_codes[:T * K].cpu().numpy(), ref.h_codes)
    assert np.array_equal(bits(layer.h_out[:T * K].cpu().numpy()), bits(ref.h))
    assert np.array_equal(bits(y), bits(want))


@pytest.mark.parametrize("H,I,E,K,T,gate_q5k", [(1024, 512, 8, 4, 9, False), (1024, 512, 8, 4, 2, False), (512, 256, 6, 2, 5, True),
                                                  (512, 256, 4, 2, 70, False), (768, 256, 1, 1, 21, False)])
def test_swiglu_clamp_trait_in_every_projection_kernel(strix, H, I, E, K, T, gate_q5k):
    """The SwiGLU clamp (include/strix/moe/activation_policy.hpp:22-24) in the 64-row sweep (9 rows), the 16-row sweep (2 rows),
    the Q5_K projection and the matrix-core sweep's epilogue (70 rows over 4 experts; a dense FFN of 21 rows): with the declared exp every bit of h, of its A8 image and of the layer output equals the oracle's,
    the limit actually binds, and gate_out / up_out keep the RAW projections."""
    rng = np.random.default_rng(H + T)
    limit = 0.02
    if gate_q5k:
        gate, up = orc.random_q5_k(rng, (E, I), H), orc.random_q5_k(rng, (E, I), H)
        down = make_layer(rng, H, I, E)[2]
    else:
        gate, up, down = make_layer(rng, H, I, E)
    gt = orc.Q5_K if gate_q5k else orc.Q4_K
    x = rng.standard_normal((T, H)).astype(np.float16)
    wr = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    ids_ref, w_ref, _, _ = orc.route(x.astype(np.float32), wr, K)
    c, d, s, _ = orc.quantize_a8(x.astype(np.float32))
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T, exp_kind=1, intermediates=True, swiglu_limit=limit,
                           gate_type=strix.TYPE_Q5_K if gate_q5k else strix.TYPE_Q4_K)
    y = layer.run(dev(x), dev(ids_ref.astype(np.int32)), dev(w_ref)).cpu().numpy()
    ref = orc.routed_experts(H, I, K, gate, up, down, orc.Q4_K, c, d, s, ids_ref, exp_kind=1, swiglu_limit=limit, gate_type=gt)
    free = orc.routed_experts(H, I, K, gate, up, down, orc.Q4_K, c, d, s, ids_ref, exp_kind=1, gate_type=gt)
    n = T * K
    assert np.array_equal(bits(layer.gate_out[:n].cpu().numpy()), bits(ref.gate)) and np.array_equal(bits(ref.gate), bits(free.gate))
    assert np.array_equal(bits(layer.up_out[:n].cpu().numpy()), bits(ref.up))
    assert np.array_equal(bits(layer.h_out[:n].cpu().numpy()), bits(ref.h)) and not np.array_equal(bits(ref.h), bits(free.h))
    assert np.array_equal(layer.down_codes[:n].cpu().numpy(), ref.h_codes) and np.array_equal(bits(layer.down_deltas[:n].cpu().numpy()), bits(ref.h_deltas))
    assert np.array_equal(bits(y), bits(orc.combine(0, w_ref, ids_ref, ref.rawdots)))
    assert np.all(layer.status[:T].cpu().numpy() == 0)
    # the dense entry of the same producer
    g_d, u_d = layer.gate_out[:n].clone(), layer.up_out[:n].clone()
    hc, hd, hs, hv, st = strix.swiglu_quantize(g_d, u_d, exp_kind=1, swiglu_limit=limit)
    assert np.array_equal(hc.cpu().numpy(), ref.h_codes) and np.array_equal(bits(hv.cpu().numpy()), bits(ref.h)) and int(st.sum()) == 0


def test_swiglu_clamp_admission(strix):
    rng = np.random.default_rng(2)
    gate, up, down = make_layer(rng, 256, 256, 2)
    x = dev(rng.standard_normal((1, 256)).astype(np.float16))
    ids, w = dev(np.zeros((1, 1), np.int32)), dev(np.ones((1, 1), np.float32))
    for bad in (-1.0, float("nan")):
        layer = strix.MoeLayer(256, 256, 2, 1, dev(gate), dev(up), dev(down), 1, swiglu_limit=bad)
        with pytest.raises(strix.StrixError) as err:
            layer.run(x, ids, w)
        assert err.value.code == strix.E_INVALID_ARGUMENT and "swiglu_limit" in str(err.value)
    for none in (0.0, float("inf")):          # 0 (the zero-initialised struct) and +infinity both mean "no clamp"
        layer = strix.MoeLayer(256, 256, 2, 1, dev(gate), dev(up), dev(down), 1, swiglu_limit=none)
        layer.run(x, ids, w)


def test_config3_moe_decode_layer_shape(strix):
    """BASELINE config 3 geometry (hidden 2048, 128 experts, top-8, intermediate 768) at 1 / 4 / 8 tokens, router included."""
    H, I, E, K = 2048, 768, 128, 8
    rng = np.random.default_rng(3)
    gate, up, down = make_layer(rng, H, I, E, full_entropy=True)
    wr = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    gd, ud, dd, wrd = dev(gate), dev(up), dev(down), dev(wr)
    layer = strix.MoeLayer(H, I, E, K, gd, ud, dd, 8, intermediates=True)
    for T in (1, 4, 8):
        x = rng.standard_normal((T, H)).astype(np.float16)
        xd = dev(x)
        ids, wts, _ = strix.route(xd, wrd, K)
        y = layer.run(xd, ids, wts).cpu().numpy()
        ids_ref, w_ref, _, _ = orc.route(x.astype(np.float32), wr, K)
        assert np.array_equal(ids.cpu().numpy().astype(np.uint32), ids_ref)          # top-k ids bit-exact
        assert np.array_equal(bits(wts.cpu().numpy()), bits(w_ref))
        c, d, s, _ = orc.quantize_a8(x.astype(np.float32))
        ref = orc.routed_experts(H, I, K, gate, up, down, orc.Q4_K, c, d, s, ids_ref)
        want = orc.combine(0, w_ref, ids_ref, ref.rawdots)
        check_layer_stages(strix, layer, y, ref, want, (c, d, s), ids_ref, w_ref, (gate, up, down, I, {}), H, K, T, 0, 0, TOL_F16)


def test_layer_entry_shared_sweeps_over_large_experts(strix):
    """A decode batch over experts whose gate + up rows exceed 4 MB (here 4.7 MB) and too large for the 16-rows-per-wavefront
    sweep (64 assignments) is planned with up to two rows per work item: every expert is chosen by several rows, so items of
    two rows and of one row both occur. Stage by stage against the oracle, through the layer entry and the staged one."""
    E, H, I, K, T = 12, 2048, 2048, 4, 16
    rng = np.random.default_rng(77)
    gate, up, down = make_layer(rng, H, I, E)
    wr = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    x = rng.standard_normal((T, H)).astype(np.float16)
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T, intermediates=True)
    ids_ref, w_ref, _, _ = orc.route(x.astype(np.float32), wr, K)
    c, d, s, _ = orc.quantize_a8(x.astype(np.float32))
    ref = orc.routed_experts(H, I, K, gate, up, down, orc.Q4_K, c, d, s, ids_ref)
    want = orc.combine(0, w_ref, ids_ref, ref.rawdots)
    y, ids, wts, _ = layer.run_layer(dev(x), dev(wr))
    assert np.array_equal(ids.cpu().numpy().astype(np.uint32), ids_ref) and np.array_equal(bits(wts.cpu().numpy()), bits(w_ref))
    items = int(layer.plan[4])
    assert T * K // 2 <= items < T * K                     # shared sweeps: fewer work items than assignments
    check_layer_stages(strix, layer, y.cpu().numpy(), ref, want, (c, d, s), ids_ref, w_ref, (gate, up, down, I, {}), H, K, T, 0, 0, TOL_F16)
    y2 = layer.run(dev(x), ids, wts)
    assert torch.equal(y2, y)


@pytest.mark.parametrize("E,K,T,bias_scale,nonfinite", [(6, 2, 200, 2.0, False), (8, 2, 40, 0.0, False), (5, 3, 97, 1.0, True)])
def test_batches_past_decode_sizes_run_the_matrix_core_sweep(strix, E, K, T, bias_scale, nonfinite):
    """Batches whose experts hold at least 4 / 16 rows on average are planned in items of 16 / 128 rows and served by the int8
    matrix-core sweep in chunks of 16 / 32 rows: a biased router makes one expert's item longer than a sweep (several chunks,
    the last one ragged and odd) while others hold a row or two. Stage by stage against the oracle - gate, up, the A8 image
    of h, rawdots bit for bit - through the layer entry and the staged one; with a non-finite weight scale in one expert the
    rows that chose it are flagged and the down stage is skipped, as on the vector-ALU sweeps."""
    H, I = 768, 512
    rng = np.random.default_rng(1000 + T)
    gate, up, down = make_layer(rng, H, I, E)
    if nonfinite:
        gate = gate.copy()
        gate.reshape(E, I, -1)[1, 7, 0:2] = np.frombuffer(np.float16(np.inf).tobytes(), np.uint8)      # d of one block of expert 1
    wr = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    bias = (rng.standard_normal(E) * bias_scale).astype(np.float32)
    x = rng.standard_normal((T, H)).astype(np.float16)
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T, intermediates=True)
    ids_ref, w_ref, _, _ = orc.route(x.astype(np.float32), wr, K, bias=bias)
    y, ids, wts, _ = layer.run_layer(dev(x), dev(wr), bias=dev(bias))
    assert np.array_equal(ids.cpu().numpy().astype(np.uint32), ids_ref) and np.array_equal(bits(wts.cpu().numpy()), bits(w_ref))
    counts = np.bincount(ids_ref.reshape(-1), minlength=E)
    split = 128 if T * K >= 16 * E else 16
    assert T * K >= 4 * E and int(layer.plan[4]) == sum(-(-int(c) // split) for c in counts)
    if bias_scale:
        assert counts.max() > 32 and counts.max() % 32 not in (0, 31)          # several chunks, a ragged last one
    if nonfinite:
        hit = np.any(ids_ref == 1, axis=1)
        st = layer.status[:T].cpu().numpy()
        assert hit.any() and not hit.all()
        assert np.all((st[hit] & strix.STATUS_NONFINITE_PROJECTION) != 0) and np.all(st[~hit] == 0)
        assert int(layer.job_status[0]) & strix.STATUS_NONFINITE_PROJECTION
        return
    c, d, s, _ = orc.quantize_a8(x.astype(np.float32))
    ref = orc.routed_experts(H, I, K, gate, up, down, orc.Q4_K, c, d, s, ids_ref)
    want = orc.combine(0, w_ref, ids_ref, ref.rawdots)
    check_layer_stages(strix, layer, y.cpu().numpy(), ref, want, (c, d, s), ids_ref, w_ref, (gate, up, down, I, {}), H, K, T, 0, 0, TOL_F16)
    y2 = layer.run(dev(x), ids, wts)
    assert torch.equal(y2, y)


@pytest.mark.parametrize("E,H,I,K,T,order", [(128, 2048, 768, 8, 8, 0), (128, 2048, 768, 8, 1, 0), (128, 2048, 768, 8, 2, 0), (160, 1536, 512, 8, 16, 0),
                                             (20, 512, 256, 3, 5, 1), (64, 1024, 256, 16, 16, 0), (160, 6144, 1280, 8, 2, 0)])
def test_whole_layer_entry_router_prologue_plan_in_one_launch(strix, E, H, I, K, T, order):
    """mi355_moe_enqueue_layer: ids / weights / scores, the A8 image, the plan-driven experts and the combine must equal
    the staged entry points bit for bit, twice in a row on the same workspace (the launch tickets return to zero). Batches of
    at most 48 assignments run the 16-rows-per-wavefront sweep in the layer entry and the 64-row sweep in the staged one."""
    rng = np.random.default_rng(E + T)
    gate, up, down = make_layer(rng, H, I, E, full_entropy=True)
    wr = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), 16)
    staged = strix.MoeLayer(H, I, E, K, layer.gate, layer.up, layer.down, 16)
    wrd = dev(wr)
    for trial in range(2):
        x = rng.standard_normal((T, H)).astype(np.float16)
        xd = dev(x)
        y, ids, wts, scores = layer.run_layer(xd, wrd, logits_order=order)
        ids_ref, w_ref, s_ref, _ = orc.route(x.astype(np.float32), wr, K, logits_order=order)
        assert np.array_equal(ids.cpu().numpy().astype(np.uint32), ids_ref)
        assert np.array_equal(bits(wts.cpu().numpy()), bits(w_ref)) and np.array_equal(bits(scores.cpu().numpy()), bits(s_ref))
        c, d, s, _ = orc.quantize_a8(x.astype(np.float32))
        assert np.array_equal(layer.codes[:T].cpu().numpy(), c) and np.array_equal(bits(layer.deltas[:T].cpu().numpy()), bits(d))
        ids2, wts2, _ = strix.route(xd, wrd, K, logits_order=order)
        assert torch.equal(ids2, ids) and torch.equal(wts2, wts)
        y2 = staged.run(xd, ids2, wts2)
        assert torch.equal(y, y2) and torch.equal(layer.rawdots[:T], staged.rawdots[:T])
        assert np.all(layer.status[:T].cpu().numpy() == 0)
        n_plan = int(strix.lib().mi355_moe_plan_words(E, 16, K))
        assert int(layer.plan[3]) == 0 and bool((layer.plan[16:272] == 0).all())      # the ticket words are left zero


def test_layer_entry_one_workspace_varying_batch_sizes(strix):
    """A decode workspace is reused with whatever batch arrives: 8 rows, then 1, 4, 2, 8 on the same MoeLayer must each
    equal a fresh staged run (the plan's ticket words sit at a place that does not depend on the row count)."""
    E, H, I, K = 128, 2048, 768, 8
    rng = np.random.default_rng(77)
    gate, up, down = make_layer(rng, H, I, E, full_entropy=True)
    wrd = dev((rng.standard_normal((E, H)) * 0.02).astype(np.float32))
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), 8)
    staged = strix.MoeLayer(H, I, E, K, layer.gate, layer.up, layer.down, 8)
    x = dev(rng.standard_normal((8, H)).astype(np.float16))
    for rows in (8, 1, 4, 2, 8):
        y, ids, wts, _ = layer.run_layer(x[:rows], wrd)
        ids2, wts2, _ = strix.route(x[:rows], wrd, K)
        assert torch.equal(ids2, ids) and torch.equal(wts2, wts)
        y2 = staged.run(x[:rows], ids2, wts2)
        assert torch.equal(y, y2) and torch.equal(layer.rawdots[:rows], staged.rawdots[:rows])
        assert np.all(layer.status[:rows].cpu().numpy() == 0) and bool((layer.plan[16:272] == 0).all())


def test_tp_rank_shard_on_the_matrix_core_sweep(strix):
    """The rank's share read in place through strides (as in config 5) at a batch that runs the matrix-core sweep: 90 rows
    over 5 experts, items of up to 128 rows; gate / up rows and down K blocks of rank 1 of 2, declared exp."""
    H, I, E, K, T = 768, 1024, 5, 2, 90
    out = run_layer_both(strix, H, I, E, K, T, seed=56, combine=1, tp=(1, 2), exp_kind=1)
    assert int(out[0].plan[4]) < T * K // 4          # grouped items, not one per assignment
    check_layer_stages(strix, *out[:7], out[7], H, K, T, 1, 1, TOL_F16)


def test_config5_tp_rank_partial_sums(strix):
    """BASELINE config 5 structure at reduced size: rank 0 of TP = 2 holds the first half of every expert's intermediate
    rows and the matching K blocks of every down row, read in place through strides; the kernel emits the rank's partial
    sums (product-then-add fold in ascending expert id), with no cross-rank reduction."""
    H, I, E, K, T = 1536, 1024, 10, 4, 16
    for rank in (0, 1):
        out = run_layer_both(strix, H, I, E, K, T, seed=55, combine=1, tp=(rank, 2))
        check_layer_stages(strix, *out[:7], out[7], H, K, T, 1, 0, TOL_F16)


@pytest.mark.parametrize("H,I,batches", [(1280, 1792, (1, 4, 5, 6, 7, 8, 11, 16)), (1024, 2048, (1, 2, 3, 4, 5, 8, 9, 12, 13))])
def test_dense_q4k_ffn_is_the_single_expert_case(strix, H, I, batches):
    """BASELINE config 2 structure at reduced size: a dense Q4_K FFN is the one-expert, top-1, weight-1 layer. The second
    shape (row lengths that are multiples of 4 super-blocks) runs the pair-per-lane dense sweep for 1 and 2 rows, the first the
    row-per-lane sweep; 3..16 rows run the int8 matrix-core sweep (each of its four widths appears); all must give the oracle's bits."""
    for T in batches:
        rng = np.random.default_rng(20 + T)
        gate, up, down = make_layer(rng, H, I, 1)
        x = rng.standard_normal((T, H)).astype(np.float16)
        ids = np.zeros((T, 1), np.int32)
        w = np.ones((T, 1), np.float32)
        layer = strix.MoeLayer(H, I, 1, 1, dev(gate), dev(up), dev(down), T, intermediates=True)
        y = layer.run(dev(x), dev(ids), dev(w)).cpu().numpy()
        c, d, s, _ = orc.quantize_a8(x.astype(np.float32))
        ref = orc.routed_experts(H, I, 1, gate, up, down, orc.Q4_K, c, d, s, ids.astype(np.uint32))
        want = orc.combine(0, w, ids.astype(np.uint32), ref.rawdots)
        check_layer_stages(strix, layer, y, ref, want, (c, d, s), ids.astype(np.uint32), w, (gate, up, down, I, {}), H, 1, T, 0, 0, TOL_F16)
        # informational: the A8 class sits ~0.5 % from the exact-weight product, which is why classes are never mixed
        g_exact = orc.base_linear(orc.Q4_K, gate[0], H // 256 * 144, I, H, x.astype(np.float32))
        assert 1e-4 < rel_err(layer.gate_out[:T].cpu().numpy(), g_exact)[0] < 5e-2


@pytest.mark.parametrize("combine", [0, 1])
@pytest.mark.parametrize("H,I,T", [(1024, 2048, 1), (1024, 2048, 2), (1024, 2048, 4), (1280, 1792, 7), (1024, 2048, 12)])
def test_dense_top1_job_publishes_its_rows_from_the_down_launch(strix, combine, H, I, T):
    """A dense top-1 job through mi355_moe_enqueue has no merge launch: the dense sweeps (pair-per-lane for 1 - 2 rows, matrix
    cores from 3) publish weight x value (+ base) with the value they computed. Output, rawdots and status words must equal the
    staged entry points' (down, then merge) bit for bit, for both combine forms, weights other than 1, a base term, and a row
    with an invalid route, which is flagged and publishes nothing."""
    import ctypes as C
    rng = np.random.default_rng(40 + T + combine)
    gate, up, down = make_layer(rng, H, I, 1)
    x = dev(rng.standard_normal((T, H)).astype(np.float16))
    ids = torch.zeros((T, 1), dtype=torch.int32, device="cuda")
    if T >= 2:
        ids[1, 0] = 3                                            # no such expert: the row is flagged, the job goes on
    w = dev((rng.standard_normal((T, 1)) * 0.7).astype(np.float32))
    base = dev(rng.standard_normal((T, H)).astype(np.float32))
    outs = []
    for staged in (False, True):
        layer = strix.MoeLayer(H, I, 1, 1, dev(gate), dev(up), dev(down), T, intermediates=True)
        layer.output.fill_(-7.0)
        if staged:
            rows, rv = layer.rows_view(x, ids, w, base)
            L, st = strix.lib(), torch.cuda.current_stream().cuda_stream
            for call in (L.mi355_moe_enqueue_prologue, L.mi355_moe_enqueue_csr, L.mi355_moe_enqueue_project, L.mi355_moe_enqueue_down):
                assert call(C.byref(layer.w), C.byref(rv), rows, C.c_void_p(st)) == 0, L.mi355_last_error()
            assert L.mi355_moe_enqueue_merge(C.byref(layer.w), C.byref(rv), rows, combine, C.c_void_p(st)) == 0, L.mi355_last_error()
        else:
            layer.run(x, ids, w, base=base, combine=combine)
        torch.cuda.synchronize()
        outs.append((layer.output[:T].clone(), layer.rawdots[:T].clone(), layer.status[:T].clone()))
    (y, raw, status), (y_s, raw_s, status_s) = outs
    assert torch.equal(status, status_s) and torch.equal(raw, raw_s)
    assert torch.equal(y.view(torch.int32), y_s.view(torch.int32))
    good = [t for t in range(T) if t != 1]
    assert all(int(status[t]) == 0 for t in good) and (T < 2 or (int(status[1]) != 0 and bool((y[1] == -7.0).all())))
    want = orc.combine(combine, w.cpu().numpy(), np.zeros((T, 1), np.uint32), raw.cpu().numpy(), base=base.cpu().numpy())
    assert np.array_equal(bits(y.cpu().numpy()[good]), bits(want[good]))


@pytest.mark.parametrize("combine", [0, 1])
@pytest.mark.parametrize("T,down_type", [(8, orc.Q4_K), (1, orc.Q4_K), (2, orc.Q4_K), (5, orc.Q4_K), (8, orc.Q8_0), (3, orc.Q8_0),
                                         (8, orc.Q6_K), (3, orc.Q6_K), (8, orc.Q5_1), (3, orc.Q5_1)])
def test_layer_entry_down_rows_and_combine_in_one_launch(strix, combine, T, down_type):
    """A decode batch whose (row, 64 columns) workgroups are all resident takes the down rows and the ordered combine in one
    launch (a wave per slot): output, rawdots and status words must equal the staged entry points' bit for bit, for both
    combine forms and with a base term. One to six rows take the same in the 16-rows-per-wavefront layout (T = 1, 2: the
    four-slot ring, T = 5: the two-slot ring); Q8_0 down rows (the host executor's format) in their four-chains-per-row layout,
    Q6_K down rows with direct loads, Q5_1 down rows through a copy ring per wave."""
    E, H, I, K = 32, 1024, 512, 8
    rng = np.random.default_rng(91 + combine + 7 * T + down_type)
    gate, up, down = make_layer(rng, H, I, E)
    if down_type == orc.Q8_0:
        down = orc.quantize_rows(orc.Q8_0, (rng.standard_normal((E, H, I)) * 0.02).astype(np.float32))
    elif down_type == orc.Q6_K:
        down = orc.random_q6_k(rng, (E, H), I)
    elif down_type == orc.Q5_1:
        down = orc.random_q5_1(rng, (E, H), I)
    x = dev(rng.standard_normal((T, H)).astype(np.float16))
    wr = dev((rng.standard_normal((E, H)) * 0.02).astype(np.float32))
    base = dev(rng.standard_normal((T, H)).astype(np.float32))
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T, down_type=down_type)
    y, ids, wts, _ = layer.run_layer(x, wr, base=base, combine=combine)
    y, raw = y.clone(), layer.rawdots[:T].clone()
    assert int(layer.status.sum()) == 0
    staged = strix.MoeLayer(H, I, E, K, layer.gate, layer.up, layer.down, T, down_type=down_type)
    want = staged.run(x, ids.clone(), wts.clone(), base=base, combine=combine)
    assert torch.equal(raw, staged.rawdots[:T]) and torch.equal(y, want)
    ids_n, w_n = ids.cpu().numpy().astype(np.uint32), wts.cpu().numpy()
    assert np.array_equal(bits(y.cpu().numpy()), bits(orc.combine(combine, w_n, ids_n, raw.cpu().numpy(), base=base.cpu().numpy())))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T", [2, 8, 20])
def test_layer_entry_input_kinds_and_output_stride(strix, dtype, T):
    """fp32 and bf16 input rows (the fp16 kind is the default of the other tests) through the whole-layer entry - quad sweep,
    row sweep with the fused down + combine, and the staged path of a larger batch - with output rows 64 floats apart from
    their width: router ids / weights and the output against the oracle on the same values, bit for bit; the padding between
    output rows is never written."""
    E, H, I, K = 16, 512, 256, 4
    rng = np.random.default_rng(5 + T)
    gate, up, down = make_layer(rng, H, I, E)
    wr = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    xt = torch.from_numpy(rng.standard_normal((T, H)).astype(np.float32)).to(getattr(torch, dtype))
    x32 = xt.to(torch.float32).numpy()                          # the values the device sees, exactly
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T, output_stride=H + 64)
    full = layer.output.as_strided((T, H + 64), (H + 64, 1))
    full.fill_(-7.0)
    y, ids, wts, _ = layer.run_layer(xt.cuda(), dev(wr))
    ids_ref, w_ref, _, _ = orc.route(x32, wr, K)
    assert np.array_equal(ids.cpu().numpy().astype(np.uint32), ids_ref) and np.array_equal(bits(wts.cpu().numpy()), bits(w_ref))
    c, d, s, _ = orc.quantize_a8(x32)
    assert np.array_equal(layer.codes[:T].cpu().numpy(), c) and np.array_equal(bits(layer.deltas[:T].cpu().numpy()), bits(d))
    raw_dev = layer.rawdots[:T].cpu().numpy()
    assert np.array_equal(bits(y.cpu().numpy()), bits(orc.combine(0, w_ref, ids_ref, raw_dev)))
    ref = orc.routed_experts(H, I, K, gate, up, down, orc.Q4_K, c, d, s, ids_ref)
    a, e = rel_err(y.cpu().numpy(), orc.combine(0, w_ref, ids_ref, ref.rawdots))
    assert a < TOL_F16 and e < TOL_F16
    assert bool((full[:, H:] == -7.0).all()) and int(layer.status.sum()) == 0


# ------------------------------------------------------------------------------------------- the expert plan
@pytest.mark.parametrize("E,K,T", [(6, 3, 5), (128, 8, 8), (128, 8, 16), (16, 4, 40), (1024, 16, 16), (1, 1, 7), (256, 8, 500), (3, 2, 300)])
def test_expert_plan_words(strix, E, K, T):
    """The plan written by mi355_moe_enqueue_csr (the stable CSR of (row, slot) by expert, src/hip_moe_q4k_a8_probe.hip:91-147):
    header counts, offsets, touched ids, order and work items against a numpy statement, for one-workgroup plans (up to 256
    assignments) and for the wave-per-expert order of larger ones; a route id out of range belongs to no expert."""
    H, I = 256, 256
    rng = np.random.default_rng(E + T)
    one = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((1, 1, H)) * 0.02).astype(np.float32))
    gate = np.ascontiguousarray(np.broadcast_to(one, (E, I, one.shape[-1])))
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(gate), dev(gate), T)
    ids = np.stack([rng.permutation(E)[:K] if E >= K else np.zeros(K, np.int64) for _ in range(T)]).astype(np.int32)
    if E > 1:
        ids[T // 2, 0] = E + 5                                   # invalid: flagged by the prologue, skipped by the plan
    x = dev(rng.standard_normal((T, H)).astype(np.float16))
    w = dev(np.ones((T, K), np.float32))
    layer.plan.fill_(-1)
    layer.plan[16:PLAN_OFFSETS_AT] = 0               # (the words that launches expect zero)
    layer.stage("csr", x, dev(ids), w)
    plan = layer.plan.cpu().numpy().view(np.uint32)
    flat = ids.reshape(-1).astype(np.int64)
    A = T * K
    # items: 8 rows of a dense matrix; one assignment at decode sizes; past them 128 / 16 rows for the matrix-core sweep when
    # the experts hold at least 16 / 4 rows on average, else 4
    split = 8 if E == 1 else (1 if T <= 16 else 128 if A >= 16 * E else 16 if A >= 4 * E else 4)
    valid = flat < E
    counts = np.bincount(flat[valid], minlength=E)
    offsets = np.concatenate([[0], np.cumsum(counts)])
    pad4 = lambda v: (v + 3) & ~3
    offsets_at = PLAN_OFFSETS_AT
    touched_at = offsets_at + pad4(E + 1)
    order_at = touched_at + pad4(E)
    items_at = order_at + pad4(A)
    touched = np.nonzero(counts)[0]
    assert plan[0] == A and plan[1] == touched.size and plan[2] == counts.max()
    assert np.array_equal(plan[offsets_at: offsets_at + E + 1], offsets)
    assert np.array_equal(plan[touched_at: touched_at + touched.size], touched)
    order = np.argsort(np.where(valid, flat, E), kind="stable")[: int(valid.sum())]
    assert np.array_equal(plan[order_at: order_at + order.size], order)
    want_items = []
    for e in touched:
        for b in range(0, counts[e], split):
            want_items.append((e, offsets[e] + b, offsets[e] + min(b + split, counts[e]), 0))
    assert plan[4] == len(want_items)
    got_items = plan[items_at: items_at + 4 * len(want_items)].reshape(-1, 4)
    assert np.array_equal(got_items, np.array(want_items, np.uint32).reshape(-1, 4))
    bound = min(A, E + A // split)
    assert np.all(plan[items_at + 4 * len(want_items): items_at + 4 * bound] == 0)     # zero records up to the launch's item bound
    assert np.all(plan[16:272] == 0)


# ------------------------------------------------------------------------------------------- the host executor's down formats
@pytest.mark.parametrize("gate_type,down_type,H,I,E,K,T,entry", [
    (orc.Q4_K, orc.Q8_0, 512, 256, 6, 3, 5, "staged"),          # the shape of the compiled reference's own whole-job check
    (orc.Q4_K, orc.Q5_1, 512, 256, 6, 3, 5, "staged"),
    (orc.Q5_K, orc.Q8_0, 512, 256, 6, 3, 5, "staged"),
    (orc.Q4_K, orc.Q8_0, 2048, 768, 128, 8, 8, "layer"),        # config 3's layer with the executor's down format
    (orc.Q4_K, orc.Q5_1, 2048, 768, 128, 8, 1, "layer"),
    (orc.Q5_K, orc.Q5_1, 2048, 768, 128, 8, 8, "layer"),
    (orc.Q5_K, orc.Q4_K, 2048, 768, 128, 8, 2, "layer"),        # Q5_K gate/up in front of Q4_K down rows
    (orc.Q4_K, orc.Q5_1, 1024, 1280, 16, 4, 40, "staged"),      # plan items of up to four assignments
    (orc.Q5_K, orc.Q8_0, 1024, 1280, 16, 4, 40, "staged"),
    (orc.Q5_K, orc.Q8_0, 768, 512, 1, 1, 6, "staged"),          # a dense layer: the plan is still built
    (orc.Q4_K, orc.Q6_K, 512, 768, 6, 3, 5, "staged"),          # Q6_K down (src/moe_a8_down_contract.cpp:147): odd block count, 2-byte aligned rows
    (orc.Q5_K, orc.Q6_K, 2048, 768, 128, 8, 8, "layer"),
    (orc.Q4_K, orc.Q6_K, 1024, 1280, 16, 4, 40, "staged"),      # five super-blocks per row: the direct-load kernel
    (orc.Q4_K, orc.Q6_K, 512, 256, 6, 3, 7, "staged"),          # one and four super-blocks per row through LDS
    (orc.Q4_K, orc.Q6_K, 512, 1024, 6, 3, 9, "layer"),
    (orc.Q4_K, orc.Q8_0, 768, 512, 5, 2, 23, "layer"),
    (orc.Q4_K, orc.Q6_K, 512, 256, 6, 2, 4, "layer")])          # one super-block per down row
def test_down_rows_in_the_host_executor_formats(strix, gate_type, down_type, H, I, E, K, T, entry):
    """The formats of the reference's host executor (src/cpu/core/routed_expert.hpp:27-28): gate/up Q4_K or Q5_K, down Q8_0 or Q5_1.
    Device rawdots == the oracle's down rows on the device's own h image, bit for bit; the combine likewise; and, when the
    compiled reference is present and the device's h codes equal the oracle's, == reference_run's rawdots bit for bit."""
    import ctypes as C
    rng = np.random.default_rng(3 * H + T + down_type + gate_type)
    gate, up, down4 = make_layer(rng, H, I, E)
    if gate_type == orc.Q5_K:
        gate, up = orc.random_q5_k(rng, (E, I), H), orc.random_q5_k(rng, (E, I), H)
    if down_type == orc.Q5_1:
        down = orc.random_q5_1(rng, (E, H), I)
    elif down_type == orc.Q6_K:
        down = orc.random_q6_k(rng, (E, H), I)
    elif down_type == orc.Q8_0:
        down = orc.quantize_rows(orc.Q8_0, (rng.standard_normal((E, H, I)) * 0.02).astype(np.float32))
    else:
        down = down4
    x = rng.standard_normal((T, H)).astype(np.float16)
    wr = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    ids_ref, w_ref, _, _ = orc.route(x.astype(np.float32), wr, K)
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T, intermediates=True, gate_type=gate_type, down_type=down_type)
    if entry == "layer":
        y, ids, wts, _ = layer.run_layer(dev(x), dev(wr))
        assert np.array_equal(ids.cpu().numpy().astype(np.uint32), ids_ref) and np.array_equal(bits(wts.cpu().numpy()), bits(w_ref))
        y = y.cpu().numpy()
    else:
        y = layer.run(dev(x), dev(ids_ref.astype(np.int32)), dev(w_ref)).cpu().numpy()
    n = T * K
    c, d, s, _ = orc.quantize_a8(x.astype(np.float32))
    ref = orc.routed_experts(H, I, K, gate, up, down, down_type, c, d, s, ids_ref, gate_type=gate_type)
    assert np.array_equal(bits(layer.gate_out[:n].cpu().numpy()), bits(ref.gate))
    assert np.array_equal(bits(layer.up_out[:n].cpu().numpy()), bits(ref.up))
    dc, dd_, ds = layer.down_codes[:n].cpu().numpy(), layer.down_deltas[:n].cpu().numpy(), layer.down_sums[:n].cpu().numpy()
    hc, hd, hs, _ = orc.quantize_a8(layer.h_out[:n].cpu().numpy(), tiny_rule=True)
    assert np.array_equal(dc, hc) and np.array_equal(bits(dd_), bits(hd)) and np.array_equal(ds, hs)
    ref_down = orc.routed_experts(H, I, K, gate, up, down, down_type, c, d, s, ids_ref, down_only_from=(dc, dd_, ds), gate_type=gate_type)
    raw_dev = layer.rawdots[:T].cpu().numpy()
    assert np.array_equal(bits(raw_dev), bits(ref_down.rawdots))
    assert np.array_equal(bits(y), bits(orc.combine(0, w_ref, ids_ref, raw_dev)))
    assert np.all(layer.status[:T].cpu().numpy() == 0)
    a, e = rel_err(y, orc.combine(0, w_ref, ids_ref, ref.rawdots))
    assert a < TOL_F16 and e < TOL_F16, (a, e)
    R = orc.ref()
    if R is not None and down_type in (orc.Q8_0, orc.Q5_1) and np.array_equal(dc, ref.h_codes) and np.array_equal(bits(dd_), bits(ref.h_deltas)):
        asg = np.array([[t, k, ids_ref[t, k]] for t in range(T) for k in range(K)], np.uint32)
        raw = np.zeros((T, K, H), np.float32)
        status = np.zeros(T, np.uint32)
        rc = R.ref_routed_expert_run_fmt(H, I, gate.ctypes.data_as(orc.u8p), up.ctypes.data_as(orc.u8p), down.ctypes.data_as(orc.u8p),
                                         int(down_type == orc.Q5_1) + 2 * int(gate_type == orc.Q5_K), c.ctypes.data_as(orc.i8p), d.ctypes.data_as(orc.f32p),
                                         s.ctypes.data_as(orc.i32p), T, asg.ctypes.data_as(orc.u32p), n, raw.ctypes.data_as(orc.f32p),
                                         C.c_uint64(K * H), status.ctypes.data_as(orc.u32p), 0, 0)
        assert rc == 0, R.ref_last_error()
        assert np.array_equal(bits(raw_dev), bits(raw))
        print("device rawdots == compiled reference_run, %d values" % raw.size)


# ------------------------------------------------------------------------------------------- failure handling
def test_invalid_route_and_nonfinite_projection_fail_closed(strix):
    H, I, E, K, T = 512, 256, 4, 2, 3
    rng = np.random.default_rng(9)
    gate, up, down = make_layer(rng, H, I, E)
    x = rng.standard_normal((T, H)).astype(np.float16)
    ids = np.array([[0, 1], [2, 9], [3, 1]], np.int32)     # row 1 names expert 9 >= E
    w = np.full((T, K), 0.5, np.float32)
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T)
    layer.output.fill_(-7.0)
    y = layer.run(dev(x), dev(ids), dev(w)).cpu().numpy()
    st = layer.status[:T].cpu().numpy()
    assert st[1] & strix.STATUS_INVALID_ROUTE and st[0] == 0 and st[2] == 0
    assert np.all(y[1] == -7.0) and np.all(y[0] != -7.0)    # the flagged row publishes nothing
    # a non-finite projection (huge activation delta, forced from the host) stops the job before the down phase
    ids[1, 1] = 0
    layer.stage("prologue", dev(x), dev(ids), dev(w))
    layer.stage("csr", dev(x), dev(ids), dev(w))
    layer.deltas[1, 3] = 3.0e38
    layer.rawdots.fill_(-3.0)
    layer.stage("project", dev(x), dev(ids), dev(w))
    layer.stage("down", dev(x), dev(ids), dev(w))
    st = layer.status[:T].cpu().numpy()
    assert st[1] & strix.STATUS_NONFINITE_PROJECTION and st[0] == 0
    assert bool((layer.rawdots == -3.0).all())


@pytest.mark.parametrize("E,H,I,K,T", [(128, 2048, 768, 8, 8), (128, 2048, 768, 8, 2), (12, 2048, 2048, 4, 16), (160, 1536, 512, 8, 16), (6, 768, 512, 2, 40)])
def test_layer_entry_halves_equal_the_whole_call(strix, E, H, I, K, T):
    """mi355_moe_enqueue_layer_front followed by mi355_moe_enqueue_layer_back is mi355_moe_enqueue_layer, bit for bit, on every
    path of the layer entry: early routes, the fused router with either sweep, shared sweeps over large experts, large batches."""
    rng = np.random.default_rng(E * T)
    gate, up, down = make_layer(rng, H, I, E, full_entropy=True)
    wr = dev((rng.standard_normal((E, H)) * 0.02).astype(np.float32))
    x = dev(rng.standard_normal((T, H)).astype(np.float16))
    whole = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T)
    halves = strix.MoeLayer(H, I, E, K, whole.gate, whole.up, whole.down, T)
    y, ids, wts, scores = whole.run_layer(x, wr)
    halves.output.fill_(-3.0)
    halves.run_layer(x, wr, half="front")
    torch.cuda.synchronize()
    assert bool((halves.output == -3.0).all())                                  # nothing is published by the front half
    y2, ids2, wts2, scores2 = halves.run_layer(x, wr, half="back")
    assert torch.equal(y2, y) and torch.equal(ids2, ids) and torch.equal(wts2, wts) and torch.equal(scores2, scores)
    assert torch.equal(halves.rawdots[:T], whole.rawdots[:T]) and torch.equal(halves.status[:T], whole.status[:T])


def early_choice(x, wr, K, amount):
    """What the early launch of the layer entry picks: plain dot products, displaced by the test knob (route_early.hpp)."""
    z = x.astype(np.float64) @ wr.astype(np.float64).T
    e = np.arange(wr.shape[0], dtype=np.uint64)
    z = z + amount * 1e-3 * ((((e * 2654435761) & 0xffffffff) >> 28).astype(np.float64) - 8.0)
    return np.argsort(-z, axis=1, kind="stable")[:, :K].astype(np.uint32)


@pytest.mark.parametrize("E,H,I,K,T,amount", [(128, 2048, 768, 8, 8, 0), (128, 2048, 768, 8, 8, 40), (128, 2048, 768, 8, 7, 400),
                                               (32, 1024, 512, 4, 16, 25), (24, 512, 256, 8, 16, 300)])
def test_layer_entry_early_routes_are_verified_and_repaired(strix, E, H, I, K, T, amount):
    """Decode batches on the 64-row sweeps pick their experts from lane-parallel logits first and run the exact router beside
    the projection. With the early logits displaced by the test knob the two choices differ in many slots: ids, weights, the
    A8 image of h, rawdots and the output must still be the exact router's, bit for bit, the work items must name the exact
    experts, and a second call on the same workspace without the displacement must give the same bits."""
    rng = np.random.default_rng(E + T + amount)
    gate, up, down = make_layer(rng, H, I, E, full_entropy=True)
    wr = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    x = rng.standard_normal((T, H)).astype(np.float16)
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T, intermediates=True)
    ids_ref, w_ref, _, _ = orc.route(x.astype(np.float32), wr, K)
    differ = int((early_choice(x, wr, K, amount) != ids_ref).sum())
    assert (differ == 0) if amount == 0 else (differ >= 3)
    c, d, s, _ = orc.quantize_a8(x.astype(np.float32))
    ref = orc.routed_experts(H, I, K, gate, up, down, orc.Q4_K, c, d, s, ids_ref)
    want = orc.combine(0, w_ref, ids_ref, ref.rawdots)
    strix.lib().mi355_debug_early_route_perturb(amount)
    try:
        y, ids, wts, _ = layer.run_layer(dev(x), dev(wr))
        y = y.clone()
        torch.cuda.synchronize()
    finally:
        strix.lib().mi355_debug_early_route_perturb(0)
    assert np.array_equal(ids.cpu().numpy().astype(np.uint32), ids_ref) and np.array_equal(bits(wts.cpu().numpy()), bits(w_ref))
    pad4 = lambda v: (v + 3) & ~3
    items_at = PLAN_OFFSETS_AT + pad4(E + 1) + pad4(E) + pad4(T * K)          # offsets, touched, order
    items = layer.plan[items_at: items_at + 4 * T * K].cpu().numpy().astype(np.uint32).reshape(-1, 4)
    assert np.array_equal(items[:, 0], ids_ref.reshape(-1))                      # the work items name the exact experts
    assert bool((layer.plan[16:272] == 0).all()) and int(layer.job_status[0]) == 0
    check_layer_stages(strix, layer, y.cpu().numpy(), ref, want, (c, d, s), ids_ref, w_ref, (gate, up, down, I, {}), H, K, T, 0, 0, TOL_F16)
    again, ids2, wts2, _ = layer.run_layer(dev(x), dev(wr))
    assert torch.equal(again, y) and torch.equal(ids2, ids) and torch.equal(wts2, wts)


@pytest.mark.parametrize("E,H,I,K,T,amount", [(128, 2048, 768, 8, 8, 10), (32, 1024, 512, 4, 16, 40)])
def test_layer_entry_repairs_reordered_slots_by_copying_their_h_image(strix, E, H, I, K, T, amount):
    """Without the optional fp32 intermediates a slot whose exact expert the early choice held under ANOTHER slot of the row is
    repaired by copying that slot's A8 image of h; only experts the early choice did not hold are swept again. Rows of both
    kinds (and rows with both at once) must leave the bits of an undisturbed call: ids, weights, the A8 image of h, rawdots
    (== the oracle's down rows on that image), the output (== the oracle's combine of them)."""
    rng = np.random.default_rng(E + T + amount + 1000)
    wr = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    x = rng.standard_normal((T, H)).astype(np.float16)
    gate, up, down = make_layer(rng, H, I, E, full_entropy=True)
    ids_ref, w_ref, _, _ = orc.route(x.astype(np.float32), wr, K)
    early = early_choice(x, wr, K, amount)
    reordered = [r for r in range(T) if set(early[r]) == set(ids_ref[r]) and (early[r] != ids_ref[r]).any()]
    replaced = [r for r in range(T) if set(early[r]) != set(ids_ref[r])]
    assert len(reordered) >= 3 and len(replaced) >= 3
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T)
    n = T * K
    snapshot = lambda: [t[:n].clone() for t in (layer.down_codes, layer.down_deltas, layer.down_sums)] + [layer.rawdots[:T].clone()]
    y0, ids0, w0, _ = layer.run_layer(dev(x), dev(wr))
    y0, ids0, w0, plain = y0.clone(), ids0.clone(), w0.clone(), snapshot()
    assert np.array_equal(ids0.cpu().numpy().astype(np.uint32), ids_ref) and np.array_equal(bits(w0.cpu().numpy()), bits(w_ref))
    c, d, s, _ = orc.quantize_a8(x.astype(np.float32))
    dc, dd_, ds = (t.cpu().numpy() for t in plain[:3])
    ref_down = orc.routed_experts(H, I, K, gate, up, down, orc.Q4_K, c, d, s, ids_ref, down_only_from=(dc, dd_, ds))
    assert np.array_equal(bits(plain[3].cpu().numpy()), bits(ref_down.rawdots))
    assert np.array_equal(bits(y0.cpu().numpy()), bits(orc.combine(0, w_ref, ids_ref, ref_down.rawdots)))
    for _ in range(3):
        strix.lib().mi355_debug_early_route_perturb(amount)
        try:
            y, ids, wts, _ = layer.run_layer(dev(x), dev(wr))
            y, ids, wts, repaired = y.clone(), ids.clone(), wts.clone(), snapshot()
            torch.cuda.synchronize()
        finally:
            strix.lib().mi355_debug_early_route_perturb(0)
        assert torch.equal(ids, ids0) and torch.equal(wts, w0)
        for got, want in zip(repaired, plain):
            assert torch.equal(got.view(torch.uint8), want.view(torch.uint8))
        assert torch.equal(y.view(torch.int32), y0.view(torch.int32))
        assert np.all(layer.status[:T].cpu().numpy() == 0) and int(layer.job_status[0]) == 0


def test_down_rows_of_a_decode_batch_give_the_same_bits_launch_after_launch(strix):
    """The down rows of a decode batch stream through two LDS slots per wave, eight waves per workgroup. A copy into a slot lands
    when its data arrives, not in the order of the wave's LDS instructions, so the slot's earlier reads have to be complete
    before the copy is issued; with only 'issued' a read now and then returned the NEXT stage's bytes (a few launches in a
    hundred, a few rows of one wave). The back half of the layer, launched 3000 times on one front half: every launch leaves the
    first one's rawdots and output."""
    E, H, I, K, T = 128, 2048, 768, 8, 7
    rng = np.random.default_rng(535)
    gate, up, down = make_layer(rng, H, I, E, full_entropy=True)
    wr = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    x = rng.standard_normal((T, H)).astype(np.float16)
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T)
    xd, wd = dev(x), dev(wr)
    y, _, _, _ = layer.run_layer(xd, wd)
    y, raw = y.clone(), layer.rawdots[:T].clone()
    layer.run_layer(xd, wd, half="front")
    bad = torch.zeros((), dtype=torch.int64, device=xd.device)
    for _ in range(3000):
        again, _, _, _ = layer.run_layer(xd, wd, half="back")
        bad += (layer.rawdots[:T].view(torch.int32) != raw.view(torch.int32)).sum() + (again.view(torch.int32) != y.view(torch.int32)).sum()
    assert int(bad) == 0


@pytest.mark.parametrize("amount", [0, 500])
def test_layer_entry_early_routes_nonfinite_flags_follow_the_exact_choice(strix, amount):
    """One expert carries a non-finite block scale. The displaced early choice sends rows to it that the exact router does not
    (and the other way round): only the rows whose EXACT experts include it may be flagged, the job word carries the
    non-finite-projection bit exactly when there is such a row, and then nothing is published."""
    E, H, I, K, T = 32, 1024, 512, 4, 16
    rng = np.random.default_rng(5 + amount)
    gate, up, down = make_layer(rng, H, I, E)
    wr = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    x = rng.standard_normal((T, H)).astype(np.float16)
    ids_ref, w_ref, _, _ = orc.route(x.astype(np.float32), wr, K)
    shift = ((((np.arange(E, dtype=np.uint64) * 2654435761) & 0xffffffff) >> 28).astype(np.int64) - 8)
    counts = np.bincount(ids_ref.reshape(-1), minlength=E)
    # an expert that the displacement favours and that some, not all, rows choose exactly; and one that no row chooses exactly
    some = [e for e in range(E) if shift[e] >= 5 and 0 < np.any(ids_ref == e, axis=1).sum() < T]
    none = [e for e in range(E) if shift[e] >= 5 and counts[e] == 0]
    for bad, expect_rows in ((some[0], True), (none[0] if none else None, False)):
        if bad is None:
            continue
        g2 = gate.copy()
        g2.reshape(E, I, -1)[bad, 3, 0:2] = np.frombuffer(np.float16(np.inf).tobytes(), np.uint8)
        layer = strix.MoeLayer(H, I, E, K, dev(g2), dev(up), dev(down), T)
        layer.output.fill_(-7.0)
        if amount:
            assert np.any(early_choice(x, wr, K, amount) == bad)                  # the early launch does send rows to it
        strix.lib().mi355_debug_early_route_perturb(amount)
        try:
            y, ids, wts, _ = layer.run_layer(dev(x), dev(wr))
            torch.cuda.synchronize()
        finally:
            strix.lib().mi355_debug_early_route_perturb(0)
        assert np.array_equal(ids.cpu().numpy().astype(np.uint32), ids_ref)
        hit = np.any(ids_ref == bad, axis=1)
        st = layer.status[:T].cpu().numpy()
        assert hit.any() == expect_rows
        assert np.all((st[hit] & strix.STATUS_NONFINITE_PROJECTION) != 0) and np.all(st[~hit] == 0)
        assert bool(int(layer.job_status[0]) & strix.STATUS_NONFINITE_PROJECTION) == expect_rows
        if expect_rows:
            assert bool((y[:T] == -7.0).all())
        else:
            c, d, s, _ = orc.quantize_a8(x.astype(np.float32))
            ref = orc.routed_experts(H, I, K, g2, up, down, orc.Q4_K, c, d, s, ids_ref)
            assert np.array_equal(bits(layer.rawdots[:T].cpu().numpy()), bits(ref.rawdots)) or rel_err(y.cpu().numpy(), orc.combine(0, w_ref, ids_ref, ref.rawdots))[0] < TOL_F16


@pytest.mark.parametrize("T", [1, 2, 8, 16])
def test_layer_entry_nonfinite_input_fails_closed(strix, T):
    """An infinite input value through the whole-layer entry: the row is flagged (activation and projection bits) and the job
    status word carries the non-finite-projection bit, so the down phase of the WHOLE job is skipped and NO row is published -
    the healthy rows keep status 0 and their previous output, and the caller must read job_status to know that. The ticket
    words are left zero and a clean call on the same workspace afterwards is unaffected."""
    E, H, I, K = 16, 512, 256, 4
    rng = np.random.default_rng(31 + T)
    gate, up, down = make_layer(rng, H, I, E)
    wrd = dev((rng.standard_normal((E, H)) * 0.02).astype(np.float32))
    x = rng.standard_normal((T, H)).astype(np.float16)
    good = dev(x.copy())
    x[T - 1, 5] = np.inf
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), 16)
    want, _, _, _ = layer.run_layer(good, wrd)
    want = want.clone()
    layer.output.fill_(-7.0)
    y, ids, wts, _ = layer.run_layer(dev(x), wrd)
    st = layer.status[:T].cpu().numpy()
    assert st[T - 1] & strix.STATUS_NONFINITE_ACTIVATION and st[T - 1] & strix.STATUS_NONFINITE_PROJECTION
    assert np.all(st[: T - 1] == 0) and bool((y[:T] == -7.0).all())          # nothing of the job is published
    assert int(layer.job_status[0]) & strix.STATUS_NONFINITE_PROJECTION
    assert bool((layer.plan[16:272] == 0).all())
    # a clean call on the same workspace afterwards is unaffected
    again, _, _, _ = layer.run_layer(good, wrd)
    assert torch.equal(again, want) and np.all(layer.status[:T].cpu().numpy() == 0)


def test_admission_failures_return_before_any_enqueue(strix):
    H, I, E, K, T = 512, 256, 4, 2, 2
    rng = np.random.default_rng(10)
    gate, up, down = make_layer(rng, H, I, E)
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T)
    x = dev(rng.standard_normal((T, H)).astype(np.float16))
    ids, w = dev(np.zeros((T, K), np.int32)), dev(np.ones((T, K), np.float32))
    layer.output.fill_(5.0)
    for field, value in (("hidden", 500), ("ffn", 100), ("top_k", 17), ("gate_type", 14), ("gate", 8)):
        saved = getattr(layer.w, field)
        setattr(layer.w, field, value)
        with pytest.raises(strix.StrixError) as err:
            layer.run(x, ids, w)
        assert err.value.code == strix.E_INVALID_ARGUMENT
        setattr(layer.w, field, saved)
    layer.w.down_type = 2
    with pytest.raises(strix.StrixError) as err:
        layer.run(x, ids, w)
    assert err.value.code == strix.E_UNSUPPORTED
    layer.w.down_type = 12
    torch.cuda.synchronize()
    assert bool((layer.output == 5.0).all())


# ------------------------------------------------------------------------------------------- prefill on the matrix cores
def exact_weight_layer(x, ids, wts, gate, up, down, H, I, K, base=None, gate_type=orc.Q4_K, down_type=orc.Q4_K):
    """Exact-weight (BASE class) evaluation of the routed experts in float64 from the decoder's fp32 weights."""
    T = x.shape[0]
    raw = np.zeros((T, K, H), np.float32)
    x64 = x.astype(np.float64)
    for e in np.unique(ids):
        wg = orc.dequant_rows(gate_type, gate[e], H).astype(np.float64)
        wu = orc.dequant_rows(gate_type, up[e], H).astype(np.float64)
        wd = orc.dequant_rows(down_type, down[e], I).astype(np.float64)
        rows, slots = np.nonzero(ids == e)
        g, u = x64[rows] @ wg.T, x64[rows] @ wu.T
        h = (g / (1.0 + np.exp(-g))) * u
        raw[rows, slots] = (h @ wd.T).astype(np.float32)
    return orc.combine(0, wts, ids, raw, base=base), raw


def random_q8_0(rng, shape_rows, width):
    """Q8_0 rows of random bytes (every code incl. -128) with small finite scales of either sign."""
    w = rng.integers(0, 256, shape_rows + (width // 32 * 34,), dtype=np.uint8)
    w[..., 1::34] = (w[..., 1::34] & 0x83) | 0x20        # |d| in [2^-7, 2^-6)
    return w


@pytest.mark.parametrize("H,I,E,K,T,gate_type,down_type,random_bytes", [
    (512, 256, 1, 1, 300, orc.Q8_0, orc.Q8_0, False),       # a dense (shared) expert: one expert, every row routed to it
    (768, 1280, 3, 2, 150, orc.Q8_0, orc.Q8_0, False),
    (256, 512, 1, 1, 129, orc.Q8_0, orc.Q8_0, True),
    (512, 512, 4, 2, 200, orc.Q8_0, orc.Q4_K, False),
    (512, 256, 4, 2, 90, orc.Q4_K, orc.Q8_0, False),
    (512, 256, 4, 2, 300, orc.Q5_K, orc.Q4_K, False),       # Q5_K (fifth bits in use): even, odd and single super-block counts
    (768, 1280, 3, 2, 150, orc.Q5_K, orc.Q5_K, False),
    (256, 512, 5, 1, 129, orc.Q4_K, orc.Q5_K, False),
    # blocks of random bytes: every factor, minimum and code value occurs and h has a heavy tail (h carried as a single fp16
    # misses the bar on these: the largest error reaches 4e-3 of the rms; as hi + lo it stays near 1e-5)
    (512, 512, 4, 2, 300, orc.Q4_K, orc.Q4_K, True),
    (1024, 768, 6, 2, 200, orc.Q5_K, orc.Q5_K, True),
    (768, 512, 3, 2, 150, orc.Q4_K, orc.Q5_K, True),
    (512, 1024, 1, 1, 140, orc.Q5_K, orc.Q8_0, True)])
def test_prefill_f16_mfma_q8_0_tensors(strix, H, I, E, K, T, gate_type, down_type, random_bytes):
    """The matrix-core prefill form with Q8_0 / Q5_K / mixed expert tensors (the always-on shared expert is experts = top_k = 1
    with weight 1) against the exact-weight product, tolerance 2e-3 as for Q4_K: max abs error over the output rms, and
    elementwise on every output above a hundredth of the rms, for the unweighted down outputs and the combined output."""
    rng = np.random.default_rng(7 * H + T)
    def tensor(qtype, rows, width):
        if random_bytes:
            w = {orc.Q8_0: random_q8_0, orc.Q4_K: random_q4k, orc.Q5_K: orc.random_q5_k}[qtype](rng, (E, rows), width)
            if qtype == orc.Q4_K:
                w[..., 1::144] &= 0x0F          # d below 2^-11: h of these products stays inside fp16
            return w
        if qtype == orc.Q5_K:
            return orc.quantize_q5_k_rows((rng.standard_normal((E, rows, width)) * 0.02).astype(np.float32))
        return orc.quantize_rows(qtype, (rng.standard_normal((E, rows, width)) * 0.02).astype(np.float32))
    gate, up, down = tensor(gate_type, I, H), tensor(gate_type, I, H), tensor(down_type, H, I)
    x = rng.standard_normal((T, H)).astype(np.float16)
    if E == 1:
        ids_ref, w_ref = np.zeros((T, 1), np.int64), np.ones((T, 1), np.float32)
    else:
        wr = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
        ids_ref, w_ref, _, _ = orc.route(x.astype(np.float32), wr, K)
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T, prefill_f16=True, gate_type=gate_type, down_type=down_type)
    y = layer.run_prefill_f16(dev(x), dev(ids_ref.astype(np.int32)), dev(w_ref)).cpu().numpy()
    want, raw_ref = exact_weight_layer(x, ids_ref, w_ref, gate, up, down, H, I, K, gate_type=gate_type, down_type=down_type)
    for got, ref in ((layer.rawdots[:T].cpu().numpy(), raw_ref), (y, want)):
        ref64 = ref.astype(np.float64)
        rms = np.sqrt(np.mean(ref64 ** 2))
        assert np.max(np.abs(got - ref64)) / rms < TOL_F16
        big = np.abs(ref64) > 1e-2 * rms
        assert np.max(np.abs(got[big] - ref64[big]) / np.abs(ref64[big])) < TOL_F16
    assert np.all(layer.status[:T].cpu().numpy() == 0)
    if E == 1:      # a top-1 layer of weight 1 without the combine: its rawdots are the combined output, bit for bit
        raw = layer.run_prefill_f16(dev(x), dev(ids_ref.astype(np.int32)), dev(w_ref), combine=strix.COMBINE_NONE)
        assert np.array_equal(bits(raw.cpu().numpy().reshape(T, H)), bits(y))
    # the integer-class entries keep refusing Q8_0 gate / up tensors
    if gate_type == orc.Q8_0:
        with pytest.raises(strix.StrixError):
            layer.run(dev(x[:1]), dev(ids_ref[:1].astype(np.int32)), dev(w_ref[:1]))


def test_prefill_f16_h_beyond_fp16_fails_closed(strix):
    """The prefill form keeps h in fp16: a row whose h leaves the fp16 range is flagged as a non-finite projection, the job's
    down phase is skipped, the merge publishes no row, and a clean call on the same buffers afterwards is unaffected."""
    H, I, E, K, T = 512, 256, 4, 2, 40
    rng = np.random.default_rng(77)
    gate, up, down = make_layer(rng, H, I, E)
    x = rng.standard_normal((T, H)).astype(np.float16)
    wr = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    ids, w, _, _ = orc.route(x.astype(np.float32), wr, K)
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T, prefill_f16=True)
    want = layer.run_prefill_f16(dev(x), dev(ids.astype(np.int32)), dev(w)).clone()
    assert int(layer.status.sum()) == 0
    loud = x.copy()
    loud[3] *= 4096.0                                       # gate and up of row 3 grow 4096-fold: h far beyond 65504
    layer.output.fill_(-7.0)
    layer.rawdots.fill_(-3.0)
    y = layer.run_prefill_f16(dev(loud), dev(ids.astype(np.int32)), dev(w))
    st = layer.status[:T].cpu().numpy()
    assert st[3] & strix.STATUS_NONFINITE_PROJECTION and np.all(np.delete(st, 3) == 0)
    assert int(layer.job_status[0]) & strix.STATUS_NONFINITE_PROJECTION
    assert bool((layer.rawdots == -3.0).all()) and bool((y == -7.0).all())
    again = layer.run_prefill_f16(dev(x), dev(ids.astype(np.int32)), dev(w))
    assert torch.equal(again, want) and int(layer.status.sum()) == 0


@pytest.mark.parametrize("H,I,E,K,T", [(512, 256, 6, 2, 300), (1024, 512, 12, 4, 77), (256, 256, 3, 1, 129), (768, 1280, 5, 2, 150),
                                       # many experts chosen by few rows each (plan items of 1 to 32 rows: token tiles with no
                                       # live row beside one that has some), 3 / 5 / 8 super-blocks per row
                                       (768, 1280, 16, 4, 60), (512, 256, 40, 8, 33), (256, 256, 24, 2, 9), (2048, 768, 64, 8, 100)])
def test_prefill_f16_mfma_matches_exact_weight_product(strix, H, I, E, K, T):
    """The fp16 MFMA prefill form against the exact-weight product: tolerance 2e-3 (fp16 activations), both as max abs
    error over the output rms and elementwise on the outputs of at least rms size; the gate / up / down tiles are checked
    through the unweighted down outputs as well as the combined output. One dense projection is also tied to the oracle's BASE-class
    routine (lane-strided fp32 sums) so that the float64 reference and the oracle agree on what "exact weight" means."""
    rng = np.random.default_rng(H + T)
    gate, up, down = make_layer(rng, H, I, E)
    x = rng.standard_normal((T, H)).astype(np.float16)
    wr = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    ids_ref, w_ref, _, _ = orc.route(x.astype(np.float32), wr, K)
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T, prefill_f16=True)
    y = layer.run_prefill_f16(dev(x), dev(ids_ref.astype(np.int32)), dev(w_ref)).cpu().numpy()
    want, raw_ref = exact_weight_layer(x, ids_ref, w_ref, gate, up, down, H, I, K)
    for got, ref in ((layer.rawdots[:T].cpu().numpy(), raw_ref), (y, want)):
        ref64 = ref.astype(np.float64)
        rms = np.sqrt(np.mean(ref64 ** 2))
        assert np.max(np.abs(got - ref64)) / rms < TOL_F16                       # max abs error over the output rms
        big = np.abs(ref64) > 1e-2 * rms                                         # elementwise relative error above a hundredth of the rms
        assert np.max(np.abs(got[big] - ref64[big]) / np.abs(ref64[big])) < TOL_F16
    assert np.all(layer.status[:T].cpu().numpy() == 0)
    e0 = int(ids_ref[0, 0])
    g_oracle = orc.base_linear(orc.Q4_K, gate[e0], H // 256 * 144, I, H, x[:4].astype(np.float32))
    g64 = x[:4].astype(np.float64) @ orc.dequant_rows(orc.Q4_K, gate[e0], H).astype(np.float64).T
    assert rel_err(g_oracle, g64.astype(np.float32))[0] < 1e-5


# ------------------------------------------------------------------------------------------- the combine operator
def _combine_operands(seed, rows, top_k, width, bf16_values):
    rng = np.random.default_rng(seed)
    eo = rng.standard_normal((rows, top_k, width)).astype(np.float32)
    base = rng.standard_normal((rows, width)).astype(np.float32)
    if bf16_values:                                    # the reference's own cases feed bfloat16 values (tests/hip_hy4_routed_tests.hip:173-174)
        eo = ((eo.view(np.uint32) + 0x8000) & 0xffff0000).astype(np.uint32).view(np.float32)
        base = ((base.view(np.uint32) + 0x8000) & 0xffff0000).astype(np.uint32).view(np.float32)
    w = rng.random((rows, top_k)).astype(np.float32)
    eo[0, 0, 0] = np.nan
    eo[rows - 1, top_k - 1, width - 1] = np.inf
    eo[0, 0, 1], eo[0, 0, 2] = 1.00390625, 1.01171875   # exact ties of the rounding
    return eo, w, base


@pytest.mark.parametrize("rows,top_k,width,bf16_values", [(5, 16, 1536, True), (5, 1, 3072, True), (3, 7, 100, False), (2, 3, 33, False),
                                                          (1, 20, 257, False), (1100, 8, 4096, False)])
def test_combine_operator_bit_exact(strix, rows, top_k, width, bf16_values):
    """mi355_moe_enqueue_combine in the bf16-steps form (weights and base bound or not, operands rounded on read or not) and
    the fma form, against the oracle (itself equal to the compiled reference's combine_ref on these forms and to the vectors
    it left in tests/golden). The last shape takes the four-columns-per-thread launch."""
    eo, w, base = _combine_operands(rows * 31 + top_k, rows, top_k, width, bf16_values)
    for has_w in (True, False):
        for has_base in (True, False):
            for rounded in (False, True):
                got = strix.combine(strix.COMBINE_BF16_STEPS, dev(eo), dev(w) if has_w else None, dev(base) if has_base else None, round_eo=rounded).cpu().numpy()
                want = orc.combine(orc.COMBINE_BF16_STEPS_ROUNDED_EO if rounded else orc.COMBINE_BF16_STEPS, w if has_w else None, None, eo, base if has_base else None)
                assert np.array_equal(bits(got), bits(want)), (has_w, has_base, rounded)
    got = strix.combine(strix.COMBINE_FMA_SLOT, dev(eo), dev(w), dev(base)).cpu().numpy()
    want = orc.combine(orc.COMBINE_FMA_SLOT, w, None, eo, base)
    nan = np.isnan(want)
    assert np.array_equal(nan, np.isnan(got)) and np.array_equal(bits(got)[~nan], bits(want)[~nan])


def test_combine_operator_golden_and_refusals(strix):
    """The vectors the compiled reference wrote, straight through the device operator; and the argument rules of the
    reference's host entry (src/moe_core/route_wave_kernel.hpp:146-147, include/strix/moe/combine.hpp:41-44)."""
    import importlib.util, os
    here = os.path.dirname(os.path.abspath(__file__))
    spec = importlib.util.spec_from_file_location("make_ref_vectors", os.path.join(here, "golden", "make_ref_vectors.py"))
    mk = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mk)
    gold = np.load(os.path.join(here, "golden", "ref_vectors.npz"))
    for case in mk.COMBINE_CASES:
        eo, w, base = mk.combine_case(*case)
        d = lambda a: None if a is None else dev(a)
        assert np.array_equal(bits(strix.combine(strix.COMBINE_BF16_STEPS, dev(eo), d(w), d(base)).cpu().numpy()), gold[f"combine_{case[0]}_bits"])
        assert np.array_equal(bits(strix.combine(strix.COMBINE_BF16_STEPS, dev(eo), d(w), d(base), round_eo=True).cpu().numpy()), gold[f"combine_{case[0]}_rounded_bits"])
    eo = dev(np.ones((2, 2, 8), np.float32))
    w = dev(np.ones((2, 2), np.float32))
    with pytest.raises(strix.StrixError, match="fma_f32 needs weights and base"):
        strix.combine(strix.COMBINE_FMA_SLOT, eo, w, None)
    with pytest.raises(strix.StrixError, match="bf16-steps form only"):
        strix.combine(strix.COMBINE_FMA_SLOT, eo, w, dev(np.ones((2, 8), np.float32)), round_eo=True)
    with pytest.raises(strix.StrixError, match="form must be"):
        strix.combine(strix.COMBINE_MULADD_ASC, eo, w, None)
    assert strix.combine(strix.COMBINE_BF16_STEPS, dev(np.ones((0, 2, 8), np.float32)), None, None).shape == (0, 8)
