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


def device_q4k(gen, rows_shape, width):
    """Random Q4_K blocks with finite, moderate fp16 d / dmin (every other bit of a block is random)."""
    w = torch.randint(0, 256, rows_shape + (width // 256, 144), dtype=torch.uint8, device="cuda", generator=gen)
    w[..., 1] = (w[..., 1] & 0x13) | 0x0C
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


def test_config2_dense_q4k_ffn_full_size(strix):
    """BASELINE config 2: Q4_K FFN 27648 x 5120 (gate, up) and 5120 x 27648 (down), 8 fp16 rows, every row checked."""
    H, I, T = 5120, 27648, 8
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
