"""The MoE block around the routed experts: the RMSNorm of the input inside the router / prologue launch
(mi355_moe_enqueue_layer_normed; the reference normalises in front of the MoE, src/ops/norm/norm.hpp:40-58, declared order
src/cpu/core/reference.cpp:86-103) and the shared expert as an always-on expert of the same launches (policy.shared_experts).
Bit for bit the oracle composition rmsnorm -> route -> A8 -> experts -> ordered combine."""
import numpy as np
import pytest
import torch

import orc
from test_gpu_parity import bits, dev, make_layer
from test_gpu_a8_contract import make_down

pytestmark = pytest.mark.gpu
DT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def layer_tensors(rng, H, I, E, gate_type, down_type):
    if gate_type == orc.Q5_K:
        gate, up = orc.random_q5_k(rng, (E, I), H), orc.random_q5_k(rng, (E, I), H)
    else:
        gate = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((E, I, H)) * 0.05).astype(np.float32))
        up = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((E, I, H)) * 0.05).astype(np.float32))
    return gate, up, make_down(rng, down_type, E, H, I)


@pytest.mark.parametrize("kind,H,I,E,K,T,scaled", [
    ("f16", 2048, 768, 128, 8, 8, True),            # config 3 with the norm in front
    ("bf16", 2048, 768, 128, 8, 1, True),
    ("f32", 1024, 512, 16, 4, 16, True),
    ("f32", 1024, 512, 16, 4, 3, False),            # unit scale (no norm weight)
    ("bf16", 256, 256, 8, 2, 5, True),              # 128 lanes in the norm's reduction (n < 512)
    ("f16", 1280, 512, 16, 4, 7, True),             # a last, partial chunk of the router chain (1280 = 2 * 512 + 256)
    ("f16", 1024, 512, 16, 4, 24, True),            # beyond the fused batch: norm launch, then the staged layer
    ("bf16", 2048, 768, 128, 8, 40, False)])
def test_rmsnorm_inside_the_layer_entry(strix, kind, H, I, E, K, T, scaled):
    rng = np.random.default_rng(H + 3 * T + E)
    gate, up, down = layer_tensors(rng, H, I, E, orc.Q4_K, orc.Q4_K)
    x_t = torch.from_numpy((rng.standard_normal((T, H)) * 3.0).astype(np.float32)).to(DT[kind])
    x32 = x_t.to(torch.float32).numpy()
    nw = (1.0 + 0.2 * rng.standard_normal(H)).astype(np.float32) if scaled else None
    wr = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    eps = 1e-6
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T, intermediates=True)
    y, ids, wts, _ = layer.run_layer(x_t.cuda(), dev(wr), norm=(dev(nw) if scaled else None, eps))
    torch.cuda.synchronize()
    want_n = orc.rmsnorm_f32(x32, nw, eps)
    assert np.array_equal(bits(layer.normed[:T].cpu().numpy()), bits(want_n))
    ids_ref, w_ref, _, _ = orc.route(want_n, wr, K)
    assert np.array_equal(ids.cpu().numpy().astype(np.uint32), ids_ref) and np.array_equal(bits(wts.cpu().numpy()), bits(w_ref))
    c, d, s, _ = orc.quantize_a8(want_n)
    assert np.array_equal(layer.codes[:T].cpu().numpy(), c) and np.array_equal(bits(layer.deltas[:T].cpu().numpy()), bits(d))
    ref = orc.routed_experts(H, I, K, gate, up, down, orc.Q4_K, c, d, s, ids_ref)
    assert np.array_equal(bits(layer.rawdots[:T].cpu().numpy()), bits(ref.rawdots))
    assert np.array_equal(bits(y.cpu().numpy()), bits(orc.combine(0, w_ref, ids_ref, ref.rawdots)))
    assert np.all(layer.status[:T].cpu().numpy() == 0)
    # the standalone kernel gives the same rows
    if kind == "f32":
        assert np.array_equal(bits(strix.rmsnorm_f32(x_t.cuda(), dev(nw) if scaled else None, eps).cpu().numpy()), bits(want_n))


@pytest.mark.parametrize("gate_type,down_type,H,I,E,K,S,T", [
    (orc.Q4_K, orc.Q4_K, 2048, 768, 128, 8, 1, 8),       # config 3 plus a shared expert: nine slots, 64 + 2 work items
    (orc.Q4_K, orc.Q4_K, 1024, 512, 16, 4, 1, 1),
    (orc.Q4_K, orc.Q4_K, 1024, 512, 16, 4, 1, 6),        # two four-row items for the shared expert, the second of two rows
    (orc.Q5_K, orc.Q8_0, 1024, 512, 16, 4, 1, 16),
    (orc.Q4_K, orc.Q6_K, 512, 768, 6, 3, 2, 5),          # two always-on experts
    (orc.Q4_K, orc.Q5_1, 1024, 384, 8, 2, 1, 9),
    (orc.Q4_K, orc.Q4_K, 1024, 512, 16, 4, 1, 24)])      # the staged path: router, plan kernel
def test_shared_expert_as_an_always_on_slot(strix, gate_type, down_type, H, I, E, K, S, T):
    rng = np.random.default_rng(H + 5 * T + S + down_type)
    gate, up, down = layer_tensors(rng, H, I, E + S, gate_type, down_type)
    x = rng.standard_normal((T, H)).astype(np.float16)
    wr = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    layer = strix.MoeLayer(H, I, E + S, K + S, dev(gate), dev(up), dev(down), T, intermediates=True, gate_type=gate_type, down_type=down_type)
    y, ids, wts, _ = layer.run_layer(dev(x), dev(wr), shared_experts=S)
    torch.cuda.synchronize()
    ids_r, w_r, _, _ = orc.route(x.astype(np.float32), wr, K)
    ids_ref = np.concatenate([ids_r, np.tile(np.arange(E, E + S, dtype=np.uint32), (T, 1))], axis=1)
    w_ref = np.concatenate([w_r, np.ones((T, S), np.float32)], axis=1)
    assert np.array_equal(ids.cpu().numpy().astype(np.uint32), ids_ref) and np.array_equal(bits(wts.cpu().numpy()), bits(w_ref))
    c, d, s, _ = orc.quantize_a8(x.astype(np.float32))
    ref = orc.routed_experts(H, I, K + S, gate, up, down, down_type, c, d, s, ids_ref, gate_type=gate_type)
    n = T * (K + S)
    assert np.array_equal(bits(layer.gate_out[:n].cpu().numpy()), bits(ref.gate))
    assert np.array_equal(layer.down_codes[:n].cpu().numpy(), ref.h_codes)
    assert np.array_equal(bits(layer.rawdots[:T].cpu().numpy()), bits(ref.rawdots))
    assert np.array_equal(bits(y.cpu().numpy()), bits(orc.combine(0, w_ref, ids_ref, ref.rawdots)))
    assert np.all(layer.status[:T].cpu().numpy() == 0)
    # the router alone writes the same rows
    ids2, w2, _ = strix.route(dev(x), dev(wr), K, shared_experts=S)
    assert np.array_equal(ids2.cpu().numpy().astype(np.uint32), ids_ref) and np.array_equal(bits(w2.cpu().numpy()), bits(w_ref))


def test_block_norm_and_shared_expert_together_and_admission(strix):
    H, I, E, K, S, T = 2048, 768, 32, 4, 1, 8
    rng = np.random.default_rng(99)
    gate, up, down = layer_tensors(rng, H, I, E + S, orc.Q4_K, orc.Q4_K)
    x = (rng.standard_normal((T, H)) * 2.0).astype(np.float16)
    nw = (1.0 + 0.2 * rng.standard_normal(H)).astype(np.float32)
    wr = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    residual = rng.standard_normal((T, H)).astype(np.float32)
    layer = strix.MoeLayer(H, I, E + S, K + S, dev(gate), dev(up), dev(down), T)
    y, ids, wts, _ = layer.run_layer(dev(x), dev(wr), shared_experts=S, norm=(dev(nw), 1e-5), base=dev(residual))
    want_n = orc.rmsnorm_f32(x.astype(np.float32), nw, 1e-5)
    ids_r, w_r, _, _ = orc.route(want_n, wr, K)
    ids_ref = np.concatenate([ids_r, np.full((T, 1), E, np.uint32)], axis=1)
    w_ref = np.concatenate([w_r, np.ones((T, 1), np.float32)], axis=1)
    c, d, s, _ = orc.quantize_a8(want_n)
    ref = orc.routed_experts(H, I, K + S, gate, up, down, orc.Q4_K, c, d, s, ids_ref)
    assert np.array_equal(bits(y.cpu().numpy()), bits(orc.combine(0, w_ref, ids_ref, ref.rawdots, base=residual)))
    # the policy and the tensors must agree on the always-on experts
    with pytest.raises(strix.StrixError):
        layer.run_layer(dev(x), dev(wr), shared_experts=0)
    with pytest.raises(strix.StrixError):
        strix.route(dev(x), dev(wr), K, shared_experts=5)


@pytest.mark.parametrize("kind,H,T", [("bf16", 2048, 8), ("f16", 2560, 3), ("f32", 300, 5), ("bf16", 4096, 40), ("f32", 256, 1)])
def test_shared_gate_bit_exact(strix, kind, H, T):
    """mi355_shared_gate against the oracle (src/hip_shared_expert_launcher.hip:624-645: thread-strided fma chains, 256-leaf halving
    tree, device expf, one division), and on the order fixtures that a wrong pairing or an unfused multiply-add changes."""
    rng = np.random.default_rng(H + T)
    x_t = torch.from_numpy((rng.standard_normal((T, H)) * 2.0).astype(np.float32)).to(DT[kind])
    w = (rng.standard_normal(H) * 0.05).astype(np.float32)
    want, _ = orc.shared_gate(x_t.to(torch.float32).numpy(), w)
    got = strix.shared_gate(x_t.cuda(), dev(w)).cpu().numpy()[:, 0]
    assert np.array_equal(bits(got), bits(want))
    # written with a stride, into a wider buffer
    wide = torch.full((T, 3), -1.0, dtype=torch.float32, device="cuda")
    strix.shared_gate(x_t.cuda(), dev(w), out=wide[:, 1:2])
    assert np.array_equal(bits(wide[:, 1].cpu().numpy()), bits(want)) and bool((wide[:, 0] == -1).all()) and bool((wide[:, 2] == -1).all())
    if kind != "f32":
        return
    sig1 = orc.shared_gate(np.ones((1, 1), np.float32), np.ones(1, np.float32))[0][0]            # sigmoid(1) as the oracle rounds it
    x1, w1 = np.ones((1, 256), np.float32), np.zeros(256, np.float32)
    w1[0], w1[1], w1[128], w1[129] = 2.0 ** 24, -(2.0 ** 24), 1.0, 1.0                            # the tree gives 1, index order 2
    x2, w2 = np.zeros((1, 512), np.float32), np.zeros(512, np.float32)
    x2[0, 0], w2[0], x2[0, 256], w2[256] = -1.0, 2.0 ** 24 + 2.0 ** 13, 2.0 ** 12 + 1.0, 2.0 ** 12 + 1.0   # fused: 1, unfused: 0
    for xs, ws in ((x1, w1), (x2, w2)):
        assert orc.shared_gate(xs, ws)[1][0] == 1.0
        assert bits(strix.shared_gate(dev(xs), dev(ws)).cpu().numpy())[0, 0] == bits(np.array([sig1], np.float32))[0]


@pytest.mark.parametrize("down_type,H,I,E,K,S,T,form", [
    (orc.Q4_K, 2048, 768, 128, 8, 1, 8, 0),        # config 3 plus a gated shared expert
    (orc.Q4_K, 1024, 512, 16, 4, 1, 3, 0),         # the one-launch down + combine of a small batch
    (orc.Q8_0, 1024, 512, 16, 4, 1, 16, 0),
    (orc.Q6_K, 512, 768, 6, 3, 2, 5, 0),           # two always-on experts, each with its own gate column
    (orc.Q5_1, 1024, 384, 8, 2, 1, 9, 1),          # the product-then-sum form
    (orc.Q4_K, 1024, 512, 16, 4, 1, 24, 0)])       # the staged path: merge launch
def test_shared_expert_with_its_sigmoid_gate(strix, down_type, H, I, E, K, S, T, form):
    """The shared expert as the reference computes it: gate = sigmoid(x . ffn_gate_inp_shexp) from mi355_shared_gate is the always-on
    slot's weight (policy.shared_slot_weights) and the slot enters the sum as acc + (gate * value)
    (src/hip_shared_expert_launcher.hip:727,779; include/strix/moe/combine.hpp:56)."""
    rng = np.random.default_rng(H + 7 * T + S + down_type)
    gate, up, down = layer_tensors(rng, H, I, E + S, orc.Q4_K, down_type)
    x = rng.standard_normal((T, H)).astype(np.float16)
    wr = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    scalar = (rng.standard_normal((S, H)) * 0.05).astype(np.float32)
    residual = rng.standard_normal((T, H)).astype(np.float32)
    gates = torch.zeros((T, S), dtype=torch.float32, device="cuda")
    for s_ in range(S):
        strix.shared_gate(dev(x), dev(scalar[s_]), out=gates[:, s_:s_ + 1])
    want_g = np.stack([orc.shared_gate(x.astype(np.float32), scalar[s_])[0] for s_ in range(S)], axis=1)
    assert np.array_equal(bits(gates.cpu().numpy()), bits(want_g))
    layer = strix.MoeLayer(H, I, E + S, K + S, dev(gate), dev(up), dev(down), T, intermediates=True, down_type=down_type)
    y, ids, wts, _ = layer.run_layer(dev(x), dev(wr), shared_experts=S, shared_slot_weights=gates, base=dev(residual), combine=form)
    torch.cuda.synchronize()
    ids_r, w_r, _, _ = orc.route(x.astype(np.float32), wr, K)
    ids_ref = np.concatenate([ids_r, np.tile(np.arange(E, E + S, dtype=np.uint32), (T, 1))], axis=1)
    w_ref = np.concatenate([w_r, want_g], axis=1)
    assert np.array_equal(ids.cpu().numpy().astype(np.uint32), ids_ref) and np.array_equal(bits(wts.cpu().numpy()), bits(w_ref))
    c, d, s, _ = orc.quantize_a8(x.astype(np.float32))
    ref = orc.routed_experts(H, I, K + S, gate, up, down, down_type, c, d, s, ids_ref)
    assert np.array_equal(bits(layer.rawdots[:T].cpu().numpy()), bits(ref.rawdots))
    assert np.array_equal(bits(y.cpu().numpy()), bits(orc.combine_shared(form, w_ref, ids_ref, ref.rawdots, S, base=residual)))
    assert np.all(layer.status[:T].cpu().numpy() == 0)


# ---------------------------------------------------------------------------------- the dense A8 profile of the shared expert
@pytest.mark.parametrize("n_in,count,rows", [(4096, 2048, 1), (2048, 4096, 3), (64, 9, 2), (8192, 40, 1), (1024, 33, 5)])
def test_dense_a8_quantiser_and_chain_product_bit_exact(strix, n_in, count, rows):
    """mi355_dense_a8_quantize and mi355_gemv_q8_0_a8_chain against the oracle (the reference's dense A8 row contract,
    src/hip_q8_rows_gemv.hpp:1155-1170; tests/dense_a8_small_reference_tests.cpp:93-104), with the reference test's scale patterns
    (zero, denormal, infinity, NaN) in some blocks and a non-finite and a tiny group in the activations."""
    rng = np.random.default_rng(n_in + count)
    w = orc.quantize_rows(orc.Q8_0, (rng.standard_normal((count, n_in)) * 0.05).astype(np.float32)).reshape(count, n_in // 32, 34)
    special = [0x0000, 0x8000, 0x0001, 0x03ff, 0x0400, 0x7bff, 0x7c00, 0xfc00, 0x7e01]      # tests/dense_a8_small_reference_tests.cpp:43-44
    for i, bits_ in enumerate(special):
        o, b = (7 * i + 1) % count, (3 * i) % (n_in // 32)
        w[o, b, 0], w[o, b, 1] = bits_ & 0xff, bits_ >> 8
    w = w.reshape(count, -1)
    x = (rng.standard_normal((rows, n_in)) * 2.0).astype(np.float32)
    x[0, 33] = np.nan                                   # block 1 of row 0: delta NaN, codes 0
    x[rows - 1, 0:32] = 2.0 ** -121                     # a tiny group: delta 1, codes 0
    c, d = strix.dense_a8_quantize(dev(x))
    c_ref, d_ref = orc.dense_a8_quantize(x)
    assert np.array_equal(c.cpu().numpy(), c_ref) and np.array_equal(bits(d.cpu().numpy()), bits(d_ref))
    assert bits(d_ref)[0, 1] == 0x7fc00000 and d_ref[rows - 1, 0] == 1.0
    y = strix.gemv_q8_0_a8_chain(dev(w), c, d, n_in, count).cpu().numpy()
    y_ref = orc.gemv_q8_0_a8_chain(w, c_ref, d_ref, n_in, count)
    assert np.array_equal(bits(y), bits(y_ref))
    assert np.all(bits(y_ref)[0] == 0x7fc00000)          # row 0: every output runs through the NaN block
    # the order fixture on the device: 64 blocks, ascending chain 0, the kernel table's lane tree 61
    blocks = 64
    cx = np.zeros((1, blocks * 32), np.int8); cx[0, ::32] = 1
    dl = np.ones((1, blocks), np.float32); dl[0, 0], dl[0, -1] = 2.0 ** 24, -(2.0 ** 24)
    wf = np.zeros((1, blocks, 34), np.uint8); wf[0, :, 1] = 0x3c; wf[0, :, 2] = 1
    wf = wf.reshape(1, -1)
    assert strix.gemv_q8_0_a8_chain(dev(wf), dev(cx), dev(dl), blocks * 32, 1).item() == 0.0
    assert strix.gemv_q8_0_a8(dev(wf), dev(cx), dev(dl), blocks * 32, 1).item() == 61.0
    with pytest.raises(strix.StrixError, match="multiple of 64"):
        strix.gemv_q8_0_a8_chain(dev(wf[:, :34]), dev(cx[:, :32]), dev(dl[:, :1]), 32, 1)


def test_shared_expert_in_the_dense_a8_profile_end_to_end(strix):
    """The reference's shared expert in its dense A8 profile, step by step (src/hip_shared_expert_launcher.hip:1084-1142): A8 image
    of the bf16 row, gate and up by the ascending chain, h = silu(gate) * up with the device expf, A8 image of h, down by the chain,
    one multiply by the sigmoid gate, stored as bfloat16 - every intermediate and the result bit for bit the oracle composition."""
    H, I, T = 2048, 1024, 3
    rng = np.random.default_rng(1142)
    q8 = lambda shape: orc.quantize_rows(orc.Q8_0, (rng.standard_normal(shape) * 0.05).astype(np.float32))
    wg, wu, wd = q8((I, H)), q8((I, H)), q8((H, I))
    scalar = (rng.standard_normal(H) * 0.05).astype(np.float32)
    x_t = torch.from_numpy(rng.standard_normal((T, H)).astype(np.float32)).to(torch.bfloat16)
    x32 = x_t.to(torch.float32).numpy()
    # device
    c, d = strix.dense_a8_quantize(x_t.cuda())
    g = strix.gemv_q8_0_a8_chain(dev(wg), c, d, H, I)
    u = strix.gemv_q8_0_a8_chain(dev(wu), c, d, H, I)
    _, _, _, h, status = strix.swiglu_quantize(g, u, exp_kind=strix.EXP_GFX1151)          # h_out: (gate / (1 + expf(-gate))) * up
    hc, hd = strix.dense_a8_quantize(h)
    down = strix.gemv_q8_0_a8_chain(dev(wd), hc, hd, I, H)
    gate = strix.shared_gate(x_t.cuda(), dev(scalar))
    out = (gate * down).to(torch.bfloat16)                                                # one multiply, then the bfloat16 store
    # oracle
    c_r, d_r = orc.dense_a8_quantize(x32)
    g_r, u_r = orc.gemv_q8_0_a8_chain(wg, c_r, d_r, H, I), orc.gemv_q8_0_a8_chain(wu, c_r, d_r, H, I)
    assert np.array_equal(bits(g.cpu().numpy()), bits(g_r)) and np.array_equal(bits(u.cpu().numpy()), bits(u_r))
    h_r = np.zeros((T, I), np.float32)
    for t in range(T):
        for grp in range(I // 32):
            sl = slice(32 * grp, 32 * grp + 32)
            ok, _, _, _, h_r[t, sl] = orc.swiglu_quantize(g_r[t, sl], u_r[t, sl], orc.EXP_GFX1151, float("inf"))
            assert ok
    assert np.array_equal(bits(h.cpu().numpy()), bits(h_r)) and int(status.sum()) == 0
    hc_r, hd_r = orc.dense_a8_quantize(h_r)
    down_r = orc.gemv_q8_0_a8_chain(wd, hc_r, hd_r, I, H)
    assert np.array_equal(bits(down.cpu().numpy()), bits(down_r))
    gate_r, _ = orc.shared_gate(x32, scalar)
    want = torch.from_numpy((gate_r[:, None] * down_r).astype(np.float32)).to(torch.bfloat16)
    assert torch.equal(out.cpu().view(torch.int16), want.view(torch.int16))
