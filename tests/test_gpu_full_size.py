"""GPU parity at the full BASELINE sizes (configs 2, 4, 5; configs 1 and 3 are covered at full size in
test_gpu_parity.py). The tensors are full-entropy Q4_K / Q8_0 blocks generated on the device; they are copied to the host
once and the CPU oracle is run on every row (configs 2, 5) or on a random subset of the 4096 rows (config 4 - a row's
result depends on no other row, so a subset checked bit for bit pins the whole batch). Every comparison is bitwise
except the end-to-end output, which also carries the stated tolerance (fp16 activations: 2e-3)."""
import numpy as np
import pytest
import torch

import orc
from test_gpu_parity import TOL_F16, bits, dev, rel_err

pytestmark = pytest.mark.gpu


def device_q4k(gen, rows_shape, width, d_bits=0x13):
    """Random Q4_K blocks with finite, moderate fp16 d / dmin (every other bit of a block is random); d_bits = 0x03 keeps d
    below 2^-11, so that h of a 4096-wide product stays far inside fp16."""
    w = torch.randint(0, 256, rows_shape + (width // 256, 144), dtype=torch.uint8, device="cuda", generator=gen)
    w[..., 1] = (w[..., 1] & d_bits) | 0x0C
    w[..., 3] = (w[..., 3] & 0x03) | 0x0C
    return w.reshape(rows_shape + (width // 256 * 144,))


def device_q8_0(gen, rows, width):
    w = torch.randint(0, 256, (rows, width // 32, 34), dtype=torch.uint8, device="cuda", generator=gen)
    w[..., 1] = (w[..., 1] & 0x03) | 0x14      # fp16 scale around 2^-10
    return w.reshape(rows, width // 32 * 34)


def check_rows(layer, y, sel, x, ids_ref, w_ref, gate, up, down, H, ffn, K, combine, base=None, **strides):
    """Oracle on rows `sel` of the batch; bitwise against the device's buffers for those rows."""
    sel = np.asarray(sel)
    xs = x[sel].astype(np.float32)
    c, d, s, _ = orc.quantize_a8(xs)
    assert np.array_equal(layer.codes.cpu().numpy()[sel], c) and np.array_equal(bits(layer.deltas.cpu().numpy()[sel]), bits(d))
    ids = np.ascontiguousarray(ids_ref[sel])
    ref = orc.routed_experts(H, ffn, K, gate, up, down, orc.Q4_K, c, d, s, ids, **strides)
    slots = (sel[:, None] * K + np.arange(K)[None, :]).reshape(-1)
    assert np.array_equal(bits(layer.gate_out.cpu().numpy()[slots]), bits(ref.gate))
    assert np.array_equal(bits(layer.up_out.cpu().numpy()[slots]), bits(ref.up))
    h_dev = layer.h_out.cpu().numpy()[slots]
    hc, hd, hs, _ = orc.quantize_a8(h_dev, tiny_rule=True)
    dc, dd, ds = (t.cpu().numpy()[slots] for t in (layer.down_codes, layer.down_deltas, layer.down_sums))
    assert np.array_equal(dc, hc) and np.array_equal(bits(dd), bits(hd)) and np.array_equal(ds, hs)
    assert np.max(np.abs(h_dev - ref.h)) <= 4e-7 * np.max(np.abs(ref.h))
    ref_down = orc.routed_experts(H, ffn, K, gate, up, down, orc.Q4_K, c, d, s, ids, down_only_from=(dc, dd, ds), **strides)
    raw_dev = layer.rawdots.cpu().numpy()[sel]
    assert np.array_equal(bits(raw_dev), bits(ref_down.rawdots))
    w = np.ascontiguousarray(w_ref[sel])
    b = None if base is None else np.ascontiguousarray(base[sel])
    assert np.array_equal(bits(y[sel]), bits(orc.combine(combine, w, ids, raw_dev, base=b)))
    want = orc.combine(combine, w, ids, ref.rawdots, base=b)
    a, e = rel_err(y[sel], want)
    assert a < TOL_F16 and e < TOL_F16, (a, e)
    assert np.all(layer.status.cpu().numpy()[sel] == 0)


@pytest.mark.parametrize("T", [1, 4, 8])
def test_config2_dense_q4k_ffn_full_size(strix, T):
    """BASELINE config 2: Q4_K FFN 27648 x 5120 (gate, up) and 5120 x 27648 (down), 1 / 4 / 8 fp16 rows (each batch size runs its
    own instantiation of the dense sweep), every row checked."""
    H, I = 5120, 27648
    gen = torch.Generator(device="cuda").manual_seed(2)
    gate, up, down = device_q4k(gen, (1, I), H), device_q4k(gen, (1, I), H), device_q4k(gen, (1, H), I)
    x = torch.randn((T, H), device="cuda", generator=gen).to(torch.float16)
    ids = torch.zeros((T, 1), dtype=torch.int32, device="cuda")
    w = torch.ones((T, 1), dtype=torch.float32, device="cuda")
    layer = strix.MoeLayer(H, I, 1, 1, gate, up, down, T, intermediates=True)
    y = layer.run(x, ids, w).cpu().numpy()
    check_rows(layer, y, np.arange(T), x.cpu().numpy(), ids.cpu().numpy().astype(np.uint32), w.cpu().numpy(),
               gate.cpu().numpy(), up.cpu().numpy(), down.cpu().numpy(), H, I, 1, 0)


def test_config5_tp_rank_shard_full_size(strix):
    """BASELINE config 5: 16 rows, hidden 6144, 160 experts top-8, intermediate 2560 split over 2 ranks; this GPU = rank 0
    (gate / up rows [0, 1280) of every expert, down K-blocks [0, 5) of every row, read in place through strides), router
    included, product-then-add fold in ascending expert id."""
    H, I, E, K, T, ranks = 6144, 2560, 160, 8, 16, 2
    ffn = I // ranks
    gen = torch.Generator(device="cuda").manual_seed(5)
    gate, up, down = device_q4k(gen, (E, I), H), device_q4k(gen, (E, I), H), device_q4k(gen, (E, H), I)
    wr = torch.randn((E, H), device="cuda", generator=gen) * 0.02
    x = torch.randn((T, H), device="cuda", generator=gen).to(torch.float16)
    grb, drb = H // 256 * 144, I // 256 * 144
    strides = dict(gate_expert_stride=I * grb, gate_row_stride=grb, down_expert_stride=H * drb, down_row_stride=drb)
    layer = strix.MoeLayer(H, ffn, E, K, gate, up, down, T, intermediates=True, **strides)
    y, ids, wts, _ = layer.run_layer(x, wr, combine=1)
    y = y.cpu().numpy()
    xn, wrn = x.cpu().numpy(), wr.cpu().numpy()
    ids_ref, w_ref, _, _ = orc.route(xn.astype(np.float32), wrn, K)
    assert np.array_equal(ids.cpu().numpy().astype(np.uint32), ids_ref) and np.array_equal(bits(wts.cpu().numpy()), bits(w_ref))
    check_rows(layer, y, np.arange(T), xn, ids_ref, w_ref, gate.cpu().numpy().reshape(-1), up.cpu().numpy().reshape(-1),
               down.cpu().numpy().reshape(-1), H, ffn, K, 1, **strides)


def test_config4_prefill_full_size(strix):
    """BASELINE config 4: 4096 rows, hidden 4096, 256 routed experts top-8 (logit bias N(0, 1.5)), intermediate 2048, Q4_K,
    plus one always-on shared expert in Q8_0 whose output enters the combine as the base. Router checked on every row;
    the expert chain on 24 random rows."""
    H, I, E, K, T = 4096, 2048, 256, 8, 4096
    gen = torch.Generator(device="cuda").manual_seed(4)
    gate, up, down = device_q4k(gen, (E, I), H), device_q4k(gen, (E, I), H), device_q4k(gen, (E, H), I)
    sg, su, sd = device_q8_0(gen, I, H), device_q8_0(gen, I, H), device_q8_0(gen, H, I)
    wr = torch.randn((E, H), device="cuda", generator=gen) * 0.02
    bias = torch.randn(E, device="cuda", generator=gen) * 1.5
    x = torch.randn((T, H), device="cuda", generator=gen).to(torch.float16)
    # shared expert: A8 image of x -> Q8_0 gate / up -> SwiGLU + A8 -> Q8_0 down
    c, d, s, _ = strix.quantize_a8(x)
    sgo, suo = strix.gemv_q8_0_a8(sg, c, d, H, I), strix.gemv_q8_0_a8(su, c, d, H, I)
    hc, hd, hs, h, hstat = strix.swiglu_quantize(sgo, suo)
    base = strix.gemv_q8_0_a8(sd, hc, hd, I, H)
    layer = strix.MoeLayer(H, I, E, K, gate, up, down, T, intermediates=True)
    y, ids, wts, _ = layer.run_layer(x, wr, bias=bias, base=base)
    y = y.cpu().numpy()
    xn = x.cpu().numpy()
    ids_ref, w_ref, _, _ = orc.route(xn.astype(np.float32), wr.cpu().numpy(), K, bias=bias.cpu().numpy())
    assert np.array_equal(ids.cpu().numpy().astype(np.uint32), ids_ref)                     # all 4096 x 8 ids
    assert np.array_equal(bits(wts.cpu().numpy()), bits(w_ref))
    assert int(hstat.sum()) == 0
    sel = np.sort(np.random.default_rng(44).choice(T, 24, replace=False))
    # shared expert on the subset (oracle dense products on the device's own h image, as for the routed experts)
    cs, ds_, _, _ = orc.quantize_a8(xn[sel].astype(np.float32))
    g_ref, _ = orc.gemv_q8_0_a8(sg.cpu().numpy(), cs, ds_, H, I)
    u_ref, _ = orc.gemv_q8_0_a8(su.cpu().numpy(), cs, ds_, H, I)
    assert np.array_equal(bits(sgo.cpu().numpy()[sel]), bits(g_ref)) and np.array_equal(bits(suo.cpu().numpy()[sel]), bits(u_ref))
    qc, qd, qs, _ = orc.quantize_a8(h.cpu().numpy()[sel], tiny_rule=True)
    assert np.array_equal(hc.cpu().numpy()[sel], qc) and np.array_equal(bits(hd.cpu().numpy()[sel]), bits(qd))
    b_ref, _ = orc.gemv_q8_0_a8(sd.cpu().numpy(), qc, qd, I, H)
    base_n = base.cpu().numpy()
    assert np.array_equal(bits(base_n[sel]), bits(b_ref))
    check_rows(layer, y, sel, xn, ids_ref, w_ref, gate.cpu().numpy(), up.cpu().numpy(), down.cpu().numpy(), H, I, K, 0, base=base_n)


def test_config4_prefill_f16_mfma_full_size(strix):
    """BASELINE config 4 in the matrix-core class: router, the Q8_0 shared expert as a one-expert prefill layer whose output is
    the base of the routed combine, the 256 Q4_K routed experts. 12 random rows are checked against the exact-weight product
    in float64 (shared expert output, unweighted routed outputs and the final rows) with the stated tolerance 2e-3, as max
    abs error over the reference rms and elementwise on the outputs of at least rms size."""
    H, I, E, K, T = 4096, 2048, 256, 8, 4096
    gen = torch.Generator(device="cuda").manual_seed(40)
    gate, up, down = device_q4k(gen, (E, I), H, 0x03), device_q4k(gen, (E, I), H, 0x03), device_q4k(gen, (E, H), I, 0x03)
    sg, su, sd = device_q8_0(gen, I, H), device_q8_0(gen, I, H), device_q8_0(gen, H, I)
    wr = torch.randn((E, H), device="cuda", generator=gen) * 0.02
    bias = torch.randn(E, device="cuda", generator=gen) * 1.5
    x = torch.randn((T, H), device="cuda", generator=gen).to(torch.float16)
    ids, wts, _ = strix.route(x, wr, K, bias=bias)
    dense = strix.MoeLayer(H, I, 1, 1, sg.reshape(1, I, -1), su.reshape(1, I, -1), sd.reshape(1, H, -1), T, prefill_f16=True,
                           gate_type=strix.TYPE_Q8_0, down_type=strix.TYPE_Q8_0)
    base = dense.run_prefill_f16(x, torch.zeros((T, 1), dtype=torch.int32, device="cuda"), torch.ones((T, 1), dtype=torch.float32, device="cuda"))
    layer = strix.MoeLayer(H, I, E, K, gate, up, down, T, prefill_f16=True)
    y = layer.run_prefill_f16(x, ids, wts, base=base).cpu().numpy()
    assert int(layer.status.sum()) == 0 and int(dense.status.sum()) == 0
    sel = np.sort(np.random.default_rng(45).choice(T, 12, replace=False))
    xs = x.cpu().numpy()[sel].astype(np.float64)
    ids_n, w_n = ids.cpu().numpy()[sel].astype(np.int64), wts.cpu().numpy()[sel]

    def ffn(rows, wg, wu, wd, qtype):
        g = rows @ orc.dequant_rows(qtype, wg, H).astype(np.float64).T
        u = rows @ orc.dequant_rows(qtype, wu, H).astype(np.float64).T
        return ((g / (1.0 + np.exp(-g))) * u) @ orc.dequant_rows(qtype, wd, I).astype(np.float64).T

    def close(got, ref):
        rms = np.sqrt(np.mean(ref ** 2))
        assert np.max(np.abs(got - ref)) / rms < TOL_F16
        big = np.abs(ref) > 1e-2 * rms
        assert np.max(np.abs(got[big] - ref[big]) / np.abs(ref[big])) < TOL_F16

    base_ref = ffn(xs, sg.cpu().numpy(), su.cpu().numpy(), sd.cpu().numpy(), orc.Q8_0)
    close(base.cpu().numpy()[sel], base_ref)
    raw_ref = np.zeros((len(sel), K, H))
    for e in np.unique(ids_n):
        r, k = np.nonzero(ids_n == e)
        raw_ref[r, k] = ffn(xs[r], gate[e].cpu().numpy(), up[e].cpu().numpy(), down[e].cpu().numpy(), orc.Q4_K)
    close(layer.rawdots.cpu().numpy()[sel], raw_ref)
    close(y[sel], base_ref + np.einsum("tk,tkh->th", w_n.astype(np.float64), raw_ref))


def test_config4_size_with_the_host_executor_formats(strix):
    """Config 4's shape (4096 rows, 256 experts top-8, 32,768 assignments in plan items of up to four) with Q5_K gate/up and
    Q8_0 down tensors, integer class: the device's gate / up rows and rawdots of 16 random rows against the oracle, bit for bit
    (rawdots on the device's own h image), and the combine of those rows."""
    H, I, E, K, T = 4096, 2048, 256, 8, 4096
    gen = torch.Generator(device="cuda").manual_seed(41)

    def blocks(rows, count, size, scale_bytes, high):
        w = torch.randint(0, 256, (rows, count, size), dtype=torch.uint8, device="cuda", generator=gen)
        for at in scale_bytes:
            w[..., at] = (w[..., at] & 0x03) | high
        return w.reshape(rows, -1)
    gate, up = (blocks(E * I, H // 256, 176, (1, 3), 0x0C).reshape(E, I, -1) for _ in range(2))
    down = blocks(E * H, I // 32, 34, (1,), 0x14).reshape(E, H, -1)
    wr = torch.randn((E, H), device="cuda", generator=gen) * 0.02
    x = torch.randn((T, H), device="cuda", generator=gen).to(torch.float16)
    layer = strix.MoeLayer(H, I, E, K, gate, up, down, T, intermediates=True, gate_type=strix.TYPE_Q5_K, down_type=strix.TYPE_Q8_0)
    y, ids, wts, _ = layer.run_layer(x, wr)
    y = y.cpu().numpy()
    assert int(layer.status.sum()) == 0
    sel = np.sort(np.random.default_rng(46).choice(T, 16, replace=False))
    xs = x.cpu().numpy()[sel].astype(np.float32)
    ids_n, w_n = ids.cpu().numpy()[sel].astype(np.uint32), wts.cpu().numpy()[sel]
    ids_ref, w_ref, _, _ = orc.route(xs, wr.cpu().numpy(), K)
    assert np.array_equal(ids_n, ids_ref) and np.array_equal(bits(w_n), bits(w_ref))
    c, d, s, _ = orc.quantize_a8(xs)
    g_np, u_np, d_np = gate.cpu().numpy(), up.cpu().numpy(), down.cpu().numpy()
    ref = orc.routed_experts(H, I, K, g_np, u_np, d_np, orc.Q8_0, c, d, s, ids_ref, gate_type=orc.Q5_K)
    slots = (sel[:, None] * K + np.arange(K)[None, :]).reshape(-1)
    assert np.array_equal(bits(layer.gate_out.cpu().numpy()[slots]), bits(ref.gate))
    assert np.array_equal(bits(layer.up_out.cpu().numpy()[slots]), bits(ref.up))
    dc, dd, ds = (t.cpu().numpy()[slots] for t in (layer.down_codes, layer.down_deltas, layer.down_sums))
    ref_down = orc.routed_experts(H, I, K, g_np, u_np, d_np, orc.Q8_0, c, d, s, ids_ref, gate_type=orc.Q5_K, down_only_from=(dc, dd, ds))
    raw_dev = layer.rawdots.cpu().numpy()[sel]
    assert np.array_equal(bits(raw_dev), bits(ref_down.rawdots))
    assert np.array_equal(bits(y[sel]), bits(orc.combine(0, w_ref, ids_ref, raw_dev)))
