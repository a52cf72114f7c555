"""The reference's A8 request / bindings entry points on the GPU (mi355_a8_enqueue_probe, _down_activation_quantize,
_down_rawdots, _down_rawdots_merge) against the CPU oracle, bit for bit, in the reference's own buffer layouts:
  probe output      [(row * top_k + slot) * 2 + which][I]   (include/strix/hip_moe_q4k_a8_probe.hpp:8-12)
  down intermediates the same buffer, h replacing the gate half  (include/strix/moe_a8_down_contract.hpp:47-49)
  rawdots           [row][slot][hidden], unweighted             (include/strix/hip_moe_a8_down.hpp:19)
  slot merge        fma chain in slot order from +0, commit test, first-error record (include/strix/moe_slot_merge.hpp:1-12,47-55)."""
import numpy as np
import pytest
import torch

import orc
from test_gpu_parity import bits, dev, make_layer

pytestmark = pytest.mark.gpu
DT = {"bf16": torch.bfloat16, "f32": torch.float32, "f16": torch.float16}


def to_input(x32, kind):
    """The stored input rows and their fp32 values as the kernels read them."""
    t = torch.from_numpy(x32).to(DT[kind])
    return t, t.to(torch.float32).numpy()


def swiglu_image(g, u, limit):
    """h and its A8 image from gate / up rows [n][I], group by group through the oracle."""
    n, I = g.shape
    h, codes = np.zeros((n, I), np.float32), np.zeros((n, I), np.int8)
    deltas, sums = np.zeros((n, I // 32), np.float32), np.zeros((n, I // 32), np.int32)
    for a in range(n):
        for grp in range(I // 32):
            sl = slice(32 * grp, 32 * grp + 32)
            ok, codes[a, sl], deltas[a, grp], sums[a, grp], h[a, sl] = orc.swiglu_quantize(g[a, sl], u[a, sl], orc.EXP_GFX1151, limit)
            assert ok
    return codes, deltas, sums, h


def make_down(rng, down_type, E, H, I):
    if down_type == orc.Q5_1:
        return orc.random_q5_1(rng, (E, H), I)
    if down_type == orc.Q6_K:
        return orc.random_q6_k(rng, (E, H), I)
    if down_type == orc.Q8_0:
        return orc.quantize_rows(orc.Q8_0, (rng.standard_normal((E, H, I)) * 0.02).astype(np.float32))
    return orc.quantize_rows(orc.Q4_K, (rng.standard_normal((E, H, I)) * 0.02).astype(np.float32))


@pytest.mark.parametrize("gate_type,kind,H,I,E,K,R", [
    (orc.Q4_K, "bf16", 2048, 768, 128, 8, 1),          # config 3's geometry, the reference's C1 form
    (orc.Q4_K, "f32", 2048, 768, 128, 8, 1),
    (orc.Q5_K, "bf16", 2048, 768, 128, 8, 1),
    (orc.Q4_K, "bf16", 2560, 1536, 64, 16, 1),         # the reference's widest C1 envelope: top-16
    (orc.Q4_K, "f16", 1024, 512, 16, 4, 4),            # logical rows: 16 items, one launch of four-row tiles
    (orc.Q4_K, "bf16", 1024, 512, 16, 6, 8),           # 48 items
    (orc.Q4_K, "bf16", 2048, 768, 128, 8, 16),         # 128 items
    (orc.Q5_K, "f32", 1024, 512, 16, 4, 16),
    (orc.Q4_K, "bf16", 4096, 2048, 8, 2, 2)])          # beyond the reference's caps
def test_probe_image_and_gate_up_rows(strix, gate_type, kind, H, I, E, K, R):
    rng = np.random.default_rng(H + I + 7 * R + gate_type)
    gate, up, _ = make_layer(rng, H, I, E)
    if gate_type == orc.Q5_K:
        gate, up = orc.random_q5_k(rng, (E, I), H), orc.random_q5_k(rng, (E, I), H)
    x_t, x32 = to_input(rng.standard_normal((R, H)).astype(np.float32), kind)
    ids = np.stack([rng.permutation(E)[:K] for _ in range(R)]).astype(np.uint32)
    p = strix.A8Decode(H, I, E, K, dev(gate), dev(up), None, rows=R, gate_type=gate_type, input_dtype=DT[kind])
    p.input.copy_(x_t)
    p.routes.copy_(torch.from_numpy(ids.astype(np.int32)))
    p.intermediates.fill_(-7.0)
    p.enqueue_probe()
    torch.cuda.synchronize()
    c, d, s, _ = orc.quantize_a8(x32)
    assert np.array_equal(p.codes.cpu().numpy(), c) and np.array_equal(bits(p.deltas.cpu().numpy()), bits(d)) and np.array_equal(p.sums.cpu().numpy(), s)
    # any tensor stands in for down: only the gate / up rows are compared
    dummy_down = np.zeros((E, H, orc.row_bytes(orc.Q8_0, I)), np.uint8)
    ref = orc.routed_experts(H, I, K, gate, up, dummy_down, orc.Q8_0, c, d, s, ids, gate_type=gate_type)
    out = p.intermediates.cpu().numpy()                        # [R][K][2][I]
    assert np.array_equal(bits(out[:, :, 0]), bits(ref.gate.reshape(R, K, I)))
    assert np.array_equal(bits(out[:, :, 1]), bits(ref.up.reshape(R, K, I)))
    assert int(p.status.item()) == 0


def test_probe_rows_in_multiples_of_32_only(strix):
    """shape.rows % 32 is the whole constraint on the intermediate size (src/moe_q4k_a8_contract.cpp:347-349): 96 rows."""
    H, I, E, K = 512, 96, 3, 2
    rng = np.random.default_rng(96)
    gate = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((E, I, H)) * 0.05).astype(np.float32))
    up = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((E, I, H)) * 0.05).astype(np.float32))
    x_t, x32 = to_input(rng.standard_normal((1, H)).astype(np.float32), "bf16")
    p = strix.A8Decode(H, I, E, K, dev(gate), dev(up), None)
    p.input.copy_(x_t)
    p.routes.copy_(torch.tensor([[2, 0]], dtype=torch.int32))
    p.enqueue_probe()
    c, d, s, _ = orc.quantize_a8(x32)
    out = p.intermediates.cpu().numpy()[0]
    for slot, e in enumerate((2, 0)):
        for which, tensor in enumerate((gate, up)):
            want = np.array([orc.q4k_row_a8(tensor[e, i], c[0], d[0], s[0]) for i in range(I)], np.float32)
            assert np.array_equal(bits(out[slot, which]), bits(want))


def test_probe_invalid_route_and_nonfinite_input_are_sticky_status_bits(strix):
    """Status bits are ORed in and stay; a step whose status word is set when the projection starts stores no gate / up row at all
    (src/hip_moe_q4k_a8_probe.hip:224-225: the projection returns on a set status)."""
    H, I, E, K = 1024, 256, 8, 2
    rng = np.random.default_rng(1)
    gate, up, _ = make_layer(rng, H, I, E)
    p = strix.A8Decode(H, I, E, K, dev(gate), dev(up), None, rows=2, input_dtype=torch.float32)
    x = rng.standard_normal((2, H)).astype(np.float32)
    p.input.copy_(torch.from_numpy(x))
    p.routes.copy_(torch.tensor([[1, E], [3, 2]], dtype=torch.int32))          # slot 1 of row 0 names no expert
    p.intermediates.fill_(-7.0)
    p.status.fill_(32)                                                          # a bit the caller already holds stays
    p.enqueue_probe()
    assert int(p.status.item()) == 32 | 1
    assert np.all(p.intermediates.cpu().numpy() == -7.0)
    p.status.zero_()
    p.enqueue_probe()
    assert int(p.status.item()) == 1 and np.all(p.intermediates.cpu().numpy() == -7.0)
    x[1, 5] = np.inf
    p.input.copy_(torch.from_numpy(x))
    p.routes.copy_(torch.tensor([[1, 0], [3, 2]], dtype=torch.int32))
    p.status.zero_()
    p.enqueue_probe()
    assert int(p.status.item()) == 2 and np.all(p.intermediates.cpu().numpy() == -7.0)
    x[1, 5] = 0.25
    p.input.copy_(torch.from_numpy(x))
    p.status.zero_()
    p.enqueue_probe()
    assert int(p.status.item()) == 0 and not np.any(p.intermediates.cpu().numpy() == -7.0)


def _poisoned_decode(strix, rng, H, I, E, K, kind):
    gate, up, _ = make_layer(rng, H, I, E)
    p = strix.A8Decode(H, I, E, K, dev(gate), dev(up), None, rows=1, input_dtype=DT[kind])
    p.codes.fill_(77); p.deltas.fill_(-3.0); p.sums.fill_(-99); p.intermediates.fill_(-7.0)
    return p, gate, up


def _image_untouched(p):
    return bool((p.codes == 77).all() and (p.deltas == -3.0).all() and (p.sums == -99).all())


@pytest.mark.parametrize("H,I,K,kind", [(2560, 640, 10, "bf16"), (2560, 640, 10, "f32"), (256, 32, 1, "bf16"), (2048, 768, 8, "f16")])
@pytest.mark.parametrize("error", ["none", "route_index", "route_weight", "input"])
def test_serial_prologue_probe(strix, H, I, K, kind, error):
    """mi355_a8_enqueue_serial_prologue_probe on the reference's own cases (tests/hip_moe_q4k_a8_probe_tests.hip:303-376: hidden 2560 x
    640 x top-10 and 256 x 32 x top-1, both input kinds, each error): the cleared words, the OVERWRITTEN status word, the image
    (stored only for a clean row) and the gate / up rows (stored only for a clean step)."""
    E = 16
    rng = np.random.default_rng(H + K + len(error))
    p, gate, up = _poisoned_decode(strix, rng, H, I, E, K, kind)
    x = rng.standard_normal((1, H)).astype(np.float32)
    ids = rng.permutation(E)[:K].astype(np.uint32)[None, :]
    weights = rng.random(K).astype(np.float32)
    if error == "route_index":
        ids[0, K - 1] = E
    if error == "route_weight":
        weights[0] = np.inf
    if error == "input":
        x[0, H - 3] = np.nan
    x_t, x32 = to_input(x, kind)
    p.input.copy_(x_t)
    p.routes.copy_(torch.from_numpy(ids.astype(np.int32)))
    clear = torch.full((H + 5,), 9.0, dtype=torch.float32, device="cuda")
    p.status.fill_(0x5a5a)                                                       # stale: the prologue overwrites it
    p.enqueue_serial_prologue_probe(clear, H, dev(weights))
    torch.cuda.synchronize()
    assert bool((clear[:H] == 0).all()) and bool((clear[H:] == 9.0).all())
    want_status = {"none": 0, "route_index": 1, "route_weight": 1, "input": 2}[error]
    assert int(p.status.item()) == want_status
    if error != "none":
        assert _image_untouched(p) and np.all(p.intermediates.cpu().numpy() == -7.0)
        return
    c, d, s, _ = orc.quantize_a8(x32)
    assert np.array_equal(p.codes.cpu().numpy(), c) and np.array_equal(bits(p.deltas.cpu().numpy()), bits(d)) and np.array_equal(p.sums.cpu().numpy(), s)
    dummy_down = np.zeros((E, H, orc.row_bytes(orc.Q8_0, I)), np.uint8)
    ref = orc.routed_experts(H, I, K, gate, up, dummy_down, orc.Q8_0, c, d, s, ids)
    out = p.intermediates.cpu().numpy()
    assert np.array_equal(bits(out[0, :, 0]), bits(ref.gate.reshape(K, I))) and np.array_equal(bits(out[0, :, 1]), bits(ref.up.reshape(K, I)))


def test_quantize_only_and_the_single_row_probe_store_rules(strix):
    """mi355_a8_enqueue_quantize_only (src/hip_moe_q4k_a8_probe.hip:540-554): the image of a clean row, status ORed into, no gate / up
    row; a row whose status is already set, whose route names no expert or that holds a non-finite value stores nothing. The
    one-row probe keeps the same rules for the image and stores no row on a flagged step."""
    H, I, E, K = 2048, 768, 32, 8
    rng = np.random.default_rng(540)
    x = rng.standard_normal((1, H)).astype(np.float32)
    ids = rng.permutation(E)[:K].astype(np.uint32)[None, :]
    for entry in ("quantize_only", "probe"):
        for case, preset, want in (("clean", 0, 0), ("held", 32, 32), ("route", 0, 1), ("route_held", 64, 65), ("input", 0, 2)):
            p, gate, up = _poisoned_decode(strix, rng, H, I, E, K, "bf16")
            xs, routes = x.copy(), ids.copy()
            if case.startswith("route"):
                routes[0, 0] = E + 7
            if case == "input":
                xs[0, 1] = -np.inf
            x_t, x32 = to_input(xs, "bf16")
            p.input.copy_(x_t)
            p.routes.copy_(torch.from_numpy(routes.astype(np.int32)))
            p.status.fill_(preset)
            getattr(p, "enqueue_" + entry)()
            torch.cuda.synchronize()
            assert int(p.status.item()) == want, (entry, case)
            out = p.intermediates.cpu().numpy()
            if case != "clean":
                assert _image_untouched(p) and np.all(out == -7.0), (entry, case)
                continue
            c, d, s, _ = orc.quantize_a8(x32)
            assert np.array_equal(p.codes.cpu().numpy(), c) and np.array_equal(bits(p.deltas.cpu().numpy()), bits(d)) and np.array_equal(p.sums.cpu().numpy(), s)
            if entry == "quantize_only":
                assert np.all(out == -7.0)
            else:
                assert not np.any(out == -7.0)
    p, _, _ = _poisoned_decode(strix, rng, H, I, E, K, "bf16")
    with pytest.raises(strix.StrixError, match="serial prologue bindings"):
        p.enqueue_serial_prologue_probe(None, 0, dev(np.ones(K, np.float32)))
    two = strix.A8Decode(H, I, E, K, p.gate, p.up, None, rows=2)
    with pytest.raises(strix.StrixError, match="one logical row"):
        strix.check(strix.lib().mi355_a8_enqueue_quantize_only(__import__("ctypes").byref(two.request(2)), __import__("ctypes").byref(two.bindings(2)), None))


def test_probe_and_down_refuse_a_bad_bundle_before_any_launch(strix):
    import ctypes as C
    H, I, E, K = 1024, 256, 8, 2
    rng = np.random.default_rng(2)
    gate, up, down = make_layer(rng, H, I, E)
    p = strix.A8Decode(H, I, E, K, dev(gate), dev(up), dev(down))
    p.intermediates.fill_(-7.0)
    p.rawdots.fill_(-7.0)
    L = strix.lib()
    q, b = p.request(), p.bindings()
    b.codes = strix.DeviceBytes(b.codes.address, b.codes.bytes - 32)             # not the exact extent
    assert L.mi355_a8_enqueue_probe(C.byref(q), C.byref(b), None) == -1
    q, b = p.request(), p.bindings()
    b.output = strix.DeviceBytes(b.gate.address, b.output.bytes)                  # the output over the gate tensor
    assert L.mi355_a8_enqueue_probe(C.byref(q), C.byref(b), None) == -1
    q, b = p.request(), p.bindings()
    q.approved_numerical_identity = b"not approved"
    assert L.mi355_a8_enqueue_probe(C.byref(q), C.byref(b), None) == -1
    dq, db = p.down_request(), p.down_bindings()
    db.rawdots = strix.DeviceBytes(db.intermediates.address, db.rawdots.bytes)
    assert L.mi355_a8_enqueue_down_rawdots(C.byref(dq), C.byref(db), 1, None) == -1
    assert L.mi355_a8_enqueue_down_activation_quantize(C.byref(dq), C.byref(db), 1, 0, None) == -1
    dq, db = p.down_request(), p.down_bindings()
    dq.swiglu_limit = -1.0
    assert L.mi355_a8_enqueue_down_rawdots(C.byref(dq), C.byref(db), 1, None) == -1
    torch.cuda.synchronize()
    assert torch.all(p.intermediates == -7.0) and torch.all(p.rawdots == -7.0) and int(p.status.item()) == 0 and torch.all(p.codes == 0)


@pytest.mark.parametrize("down_type,H,I,E,K,R,limit", [
    (orc.Q4_K, 2048, 768, 128, 8, 1, float("inf")),
    (orc.Q4_K, 2048, 768, 128, 8, 1, 0.05),            # the clamped producer (src/moe_a8_down_contract.cpp:57)
    (orc.Q6_K, 2048, 768, 128, 8, 1, float("inf")),
    (orc.Q5_1, 2048, 640, 128, 8, 1, float("inf")),    # the incumbent classes: intermediate % 128
    (orc.Q8_0, 2048, 640, 128, 8, 1, 0.05),
    (orc.Q4_K, 2560, 1536, 64, 16, 1, float("inf")),
    (orc.Q4_K, 1024, 512, 16, 4, 4, float("inf")),
    (orc.Q6_K, 1024, 512, 16, 6, 8, 0.05),
    (orc.Q8_0, 1024, 384, 16, 4, 16, float("inf")),
    (orc.Q5_1, 1024, 384, 16, 4, 16, float("inf")),
    (orc.Q4_K, 2048, 768, 128, 8, 16, float("inf"))])
def test_whole_pipeline_probe_activation_rawdots(strix, down_type, H, I, E, K, R, limit):
    """probe -> down_activation_quantize -> down_rawdots: every stage bit for bit the oracle's (h and its image from the
    device's gate / up rows, the down rows from the device's image), and the oracle end to end."""
    rng = np.random.default_rng(H + I + 13 * R + down_type)
    if I % 256 == 0:
        gate, up, _ = make_layer(rng, H, I, E)
    else:
        gate = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((E, I, H)) * 0.05).astype(np.float32))
        up = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((E, I, H)) * 0.05).astype(np.float32))
    down = make_down(rng, down_type, E, H, I)
    x_t, x32 = to_input(rng.standard_normal((R, H)).astype(np.float32), "bf16")
    ids = np.stack([rng.permutation(E)[:K] for _ in range(R)]).astype(np.uint32)
    p = strix.A8Decode(H, I, E, K, dev(gate), dev(up), dev(down), rows=R, down_type=down_type, swiglu_limit=limit)
    p.input.copy_(x_t)
    p.routes.copy_(torch.from_numpy(ids.astype(np.int32)))
    p.enqueue_probe()
    gu = p.intermediates.cpu().numpy().copy()
    p.enqueue_down_activation_quantize()
    p.enqueue_down_rawdots()
    torch.cuda.synchronize()
    assert int(p.status.item()) == 0 and int(p.aggregate.item()) == 0
    after = p.intermediates.cpu().numpy()
    assert np.array_equal(bits(after[:, :, 1]), bits(gu[:, :, 1]))              # the producer replaces only the gate half
    n = R * K
    hc, hd, hs, h = swiglu_image(gu[:, :, 0].reshape(n, I), gu[:, :, 1].reshape(n, I), limit)
    assert np.array_equal(bits(after[:, :, 0].reshape(n, I)), bits(h))
    dc, dd, ds = p.h_codes.cpu().numpy().reshape(n, I), p.h_deltas.cpu().numpy().reshape(n, -1), p.h_sums.cpu().numpy().reshape(n, -1)
    assert np.array_equal(dc, hc) and np.array_equal(bits(dd), bits(hd)) and np.array_equal(ds, hs)
    c, d, s, _ = orc.quantize_a8(x32)
    ref = orc.routed_experts(H, I, K, gate, up, down, down_type, c, d, s, ids, swiglu_limit=limit)
    assert np.array_equal(bits(gu[:, :, 0].reshape(n, I)), bits(ref.gate)) and np.array_equal(bits(gu[:, :, 1].reshape(n, I)), bits(ref.up))
    assert np.array_equal(dc, ref.h_codes) and np.array_equal(bits(dd), bits(ref.h_deltas))
    assert np.array_equal(bits(p.rawdots.cpu().numpy()), bits(ref.rawdots))
    if limit != float("inf"):
        assert np.any(np.abs(gu) > limit)                                        # the clamp acted


def test_down_producer_flags_nonfinite_and_invalid_routes(strix):
    H, I, E, K = 1024, 256, 8, 2
    rng = np.random.default_rng(3)
    gate, up, down = make_layer(rng, H, I, E)
    p = strix.A8Decode(H, I, E, K, dev(gate), dev(up), dev(down))
    g = rng.standard_normal((1, K, 2, I)).astype(np.float32)
    g[0, 1, 1, 40] = np.nan
    p.intermediates.copy_(torch.from_numpy(g))
    p.routes.copy_(torch.tensor([[1, 2]], dtype=torch.int32))
    p.rawdots.fill_(-7.0)
    p.enqueue_down_activation_quantize()
    assert int(p.status.item()) == 8 and int(p.aggregate.item()) == 16
    p.enqueue_down_rawdots()                                                     # a flagged step computes no down rows
    assert torch.all(p.rawdots == -7.0)
    p.status.zero_()
    p.aggregate.zero_()
    p.intermediates.copy_(torch.from_numpy(rng.standard_normal((1, K, 2, I)).astype(np.float32)))
    p.routes.copy_(torch.tensor([[1, E + 3]], dtype=torch.int32))
    p.enqueue_down_activation_quantize()
    assert int(p.status.item()) == 1 and int(p.aggregate.item()) == 16
    # the aggregate word is optional
    p.status.zero_()
    import ctypes as C
    q, b = p.down_request(), p.down_bindings(aggregate=False)
    assert strix.lib().mi355_a8_enqueue_down_activation_quantize(C.byref(q), C.byref(b), 1, 0, None) == 0
    assert int(p.status.item()) == 1


def merge_oracle(raw, w, bf16_commit):
    """Slot merge of one row (include/strix/moe_slot_merge.hpp:1-12): +0 seed, fma per slot in order; commit test on the bits."""
    acc = orc.combine(0, w[None], np.zeros((1, w.size), np.uint32), raw[None])[0]
    failed = bool(np.any((bits(acc) & 0x7fffffff) >= (0x7f7f8000 if bf16_commit else 0x7f800000)))
    return acc, failed


@pytest.mark.parametrize("down_type,out_dtype,bf16_commit", [(orc.Q4_K, torch.float32, False), (orc.Q4_K, torch.bfloat16, True),
                                                              (orc.Q6_K, torch.bfloat16, True), (orc.Q8_0, torch.float32, False),
                                                              (orc.Q5_1, torch.bfloat16, False)])
def test_rawdots_with_slot_merge_tail(strix, down_type, out_dtype, bf16_commit):
    H, I, E, K = 2048, 768 if down_type in (orc.Q4_K, orc.Q6_K) else 640, 128, 8
    rng = np.random.default_rng(40 + down_type)
    gate = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((E, I, H)) * 0.05).astype(np.float32))
    up = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((E, I, H)) * 0.05).astype(np.float32))
    down = make_down(rng, down_type, E, H, I)
    p = strix.A8Decode(H, I, E, K, dev(gate), dev(up), dev(down), down_type=down_type)
    x_t, _ = to_input(rng.standard_normal((1, H)).astype(np.float32), "bf16")
    ids = rng.permutation(E)[:K].astype(np.int32)
    w = rng.random(K).astype(np.float32)
    w /= w.sum()
    p.input.copy_(x_t)
    p.routes.copy_(torch.from_numpy(ids[None]))
    acc, out = torch.full((H,), -3.0, device="cuda"), torch.full((H,), -3.0, device="cuda").to(out_dtype)
    record = torch.zeros(2, dtype=torch.int32, device="cuda")
    p.enqueue_probe()
    p.enqueue_down_activation_quantize()
    p.enqueue_down_rawdots_merge(dev(w), acc, out, record, domain=5, bf16_commit=bf16_commit)
    torch.cuda.synchronize()
    raw = p.rawdots.cpu().numpy()[0]
    want, failed = merge_oracle(raw, w, bf16_commit)
    assert not failed and int(p.status.item()) == 0 and record.tolist() == [0, 0]
    assert np.array_equal(bits(acc.cpu().numpy()), bits(want))
    if out_dtype == torch.float32:
        assert np.array_equal(bits(out.cpu().numpy()), bits(want))
    else:
        assert torch.equal(out.cpu(), torch.from_numpy(want).to(torch.bfloat16))          # round to nearest even
    # the same rawdots through mi355_a8_enqueue_down_rawdots
    p.rawdots.fill_(0)
    p.enqueue_down_rawdots()
    assert np.array_equal(bits(p.rawdots.cpu().numpy()[0]), bits(raw))


@pytest.mark.parametrize("down_type", [orc.Q4_K, orc.Q8_0, orc.Q6_K])
def test_rawdots_and_slot_merge_flag_an_invalid_route_on_their_own(strix, down_type):
    """A route out of range reaches the down rows without the producer that checks the routes (the routes are overwritten after
    a valid producer run and the status word is clear): mi355_a8_enqueue_down_rawdots sets the invalid-route bit and the summary
    word itself, as the reference's down_rawdots_rows does (src/hip_moe_q4k_a8_probe.hip:743); with the slot-merge tail nothing
    is accumulated or committed and the first-error record is set - also when the status word is cleared between the two."""
    H, I, E, K = 1024, 256 if down_type != orc.Q8_0 else 384, 8, 4
    rng = np.random.default_rng(90 + down_type)
    gate = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((E, I, H)) * 0.05).astype(np.float32))
    down = make_down(rng, down_type, E, H, I)
    p = strix.A8Decode(H, I, E, K, dev(gate), dev(gate), dev(down), down_type=down_type)
    p.intermediates.copy_(torch.from_numpy(rng.standard_normal((1, K, 2, I)).astype(np.float32)))
    p.routes.copy_(torch.tensor([[1, 2, 5, 7]], dtype=torch.int32))
    p.enqueue_down_activation_quantize()
    p.enqueue_down_rawdots()
    torch.cuda.synchronize()
    assert int(p.status.item()) == 0 and int(p.aggregate.item()) == 0
    good = p.rawdots.clone()
    p.routes.copy_(torch.tensor([[1, E + 3, 5, 7]], dtype=torch.int32))
    p.rawdots.fill_(-7.0)
    p.enqueue_down_rawdots()
    torch.cuda.synchronize()
    assert int(p.status.item()) == 1 and int(p.aggregate.item()) == 16
    raw = p.rawdots.cpu()
    assert torch.all(raw[0, 1] == -7.0) and torch.equal(raw[0, 0], good[0, 0].cpu()) and torch.equal(raw[0, 3], good[0, 3].cpu())
    # the merge tail: a cleared status word, the invalid route still there
    for clear_between in (False, True):
        p.status.zero_()
        p.aggregate.zero_()
        acc, out = torch.full((H,), 5.0, device="cuda"), torch.full((H,), -3.0, device="cuda")
        record = torch.zeros(2, dtype=torch.int32, device="cuda")
        w = dev(np.full(K, 0.25, np.float32))
        if clear_between:
            p.enqueue_down_rawdots()
            p.status.zero_()
        p.enqueue_down_rawdots_merge(w, acc, out, record, domain=6, bf16_commit=False)
        torch.cuda.synchronize()
        assert int(p.status.item()) & 1 and record.tolist() == [6, int(p.status.item())]
        assert torch.all(out == -3.0) and torch.all(acc == 5.0)                  # nothing accumulated, nothing committed


def test_slot_merge_commit_threshold_and_first_error_record(strix):
    """A merged value that is finite in fp32 but rounds to bf16 infinity (bits >= 0x7f7f8000) fails a bf16 commit and passes an
    fp32 one; a failed step stores no output and the record keeps the FIRST failure of the stream
    (include/strix/moe_slot_merge.hpp:47-55, include/strix/deferred_moe_status.hpp:19-26)."""
    H, I, E, K = 256, 256, 2, 2
    rng = np.random.default_rng(77)
    # a Q8_0 down tensor with huge scales: rawdots of the order 1e38 * small
    down = orc.quantize_rows(orc.Q8_0, (rng.standard_normal((E, H, I))).astype(np.float32))
    gate = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((E, I, H)) * 0.05).astype(np.float32))
    p = strix.A8Decode(H, I, E, K, dev(gate), dev(gate), dev(down), down_type=orc.Q8_0)
    p.routes.copy_(torch.tensor([[0, 1]], dtype=torch.int32))
    inter = rng.standard_normal((1, K, 2, I)).astype(np.float32)
    p.intermediates.copy_(torch.from_numpy(inter))
    p.enqueue_down_activation_quantize()
    p.enqueue_down_rawdots()
    raw = p.rawdots.cpu().numpy()[0]
    big = np.float32(np.abs(raw).max())
    # weights that scale the largest value to just below fp32 infinity but above the largest bf16
    target = np.float32(3.4e38)
    w = np.array([target / big, 0.0], np.float32)
    where = np.unravel_index(np.abs(raw).argmax(), raw.shape)
    if where[0] == 1:
        w = w[::-1].copy()
    want, failed32 = merge_oracle(raw, w, False)
    _, failed16 = merge_oracle(raw, w, True)
    assert not failed32 and failed16, "the case must sit between the two thresholds"
    acc = torch.zeros(H, device="cuda")
    out32, out16 = torch.full((H,), -3.0, device="cuda"), torch.full((H,), -3.0, device="cuda").to(torch.bfloat16)
    record = torch.zeros(2, dtype=torch.int32, device="cuda")
    p.enqueue_down_rawdots_merge(dev(w), acc, out32, record, domain=3, bf16_commit=False)
    assert int(p.status.item()) == 0 and record.tolist() == [0, 0]
    assert np.array_equal(bits(out32.cpu().numpy()), bits(want))
    p.enqueue_down_rawdots_merge(dev(w), acc, out16, record, domain=4, bf16_commit=True)
    assert int(p.status.item()) == 8 and record.tolist() == [4, 8]
    assert torch.all(out16 == -3.0)                                              # nothing committed
    assert np.array_equal(bits(acc.cpu().numpy()), bits(want))                   # the accumulation was written before the test
    # a later failure of another domain does not replace the first record; a flagged step writes nothing at all
    acc.fill_(5.0)
    p.enqueue_down_rawdots_merge(dev(w), acc, out32, record, domain=9, bf16_commit=False)
    assert record.tolist() == [4, 8] and torch.all(acc == 5.0)
