"""The union rows form of the A8 entry points (mi355_a8_enqueue_probe_union, _down_activation_quantize_union, _down_rawdots_union)
on the GPU, after the reference's device test (tests/hip_moe_a8_union_tests.hip): for R rows that share experts every buffer
must hold, byte for byte, what R single-row calls write (A8 codes, gate / up intermediates, h and its image, raw dots), the
device plan must equal the host reference of include/strix/moe/expert_union.hpp:34-57, and an expert named twice by one row
sets exactly the invalid-route bit. The single-row form itself is checked against the oracle in test_gpu_a8_contract.py; here
one case is also compared with the oracle directly."""
import numpy as np
import pytest
import torch

import orc
from test_gpu_a8_contract import make_down
from test_gpu_parity import bits, dev, make_layer

pytestmark = pytest.mark.gpu


def shared_ids(R, K, E):
    """The reference test's routes: distinct within a row, shared across rows (tests/hip_moe_a8_union_tests.hip:117-119)."""
    return np.array([[(k * 5 + r * 3) % E for k in range(K)] for r in range(R)], np.uint32)


def run_paths(strix, rng, H, I, E, K, R, down_type, ids, gate, up, down, limit=float("inf"), kind=torch.float32):
    """(single-row path run R times, union path) on the same inputs."""
    x = torch.from_numpy((rng.standard_normal((R, H)) * 1.5).astype(np.float32)).to(kind)
    c1 = strix.A8Decode(H, I, E, K, dev(gate), dev(up), dev(down), rows=1, down_type=down_type, input_dtype=kind, swiglu_limit=limit)
    un = strix.A8Decode(H, I, E, K, c1.gate, c1.up, c1.down, rows=R, down_type=down_type, input_dtype=kind, swiglu_limit=limit)
    un.input.copy_(x)
    un.routes.copy_(torch.from_numpy(ids.astype(np.int32)))
    un.enqueue_probe_union()
    un.enqueue_down_activation_quantize_union()
    un.enqueue_down_rawdots_union()
    torch.cuda.synchronize()
    rows = []
    for r in range(R):
        c1.input.copy_(x[r:r + 1])
        c1.routes.copy_(torch.from_numpy(ids[r:r + 1].astype(np.int32)))
        c1.enqueue_probe()
        c1.enqueue_down_activation_quantize()
        c1.enqueue_down_rawdots()
        torch.cuda.synchronize()
        assert int(c1.status.item()) == 0
        rows.append({n: getattr(c1, n).cpu().numpy().copy() for n in FIELDS})
    return rows, un, x


FIELDS = ("codes", "deltas", "sums", "intermediates", "h_codes", "h_deltas", "h_sums", "rawdots")


@pytest.mark.parametrize("H,I,E,K,R,down_type", [
    (1536, 1536, 64, 16, 1, orc.Q6_K),         # the reference test's geometry (Hy4 preset) and row counts
    (1536, 1536, 64, 16, 2, orc.Q6_K),
    (1536, 1536, 64, 16, 3, orc.Q6_K),
    (1536, 1536, 64, 16, 8, orc.Q6_K),
    (1536, 1536, 64, 16, 8, orc.Q4_K),
    (2048, 768, 128, 8, 5, orc.Q4_K),          # config 3's geometry: hidden past the reference's 1536
    (1024, 512, 16, 4, 8, orc.Q4_K)])          # eight rows over 16 experts: every entry is held by several rows
def test_union_rows_equal_single_row_calls_bit_for_bit(strix, H, I, E, K, R, down_type):
    rng = np.random.default_rng(H + I + R + down_type)
    gate, up, _ = make_layer(rng, H, I, E)
    down = make_down(rng, down_type, E, H, I)
    # (elsewhere: every row draws from a pool of 2 K experts, so entries are held by several rows)
    ids = shared_ids(R, K, E) if E == 64 else np.stack([rng.permutation(min(E, 2 * K))[:K] for _ in range(R)]).astype(np.uint32)
    rows, un, _ = run_paths(strix, rng, H, I, E, K, R, down_type, ids, gate, up, down, limit=10.0)
    assert int(un.status.item()) == 0
    entries = orc.expert_union_build(ids, R, K, E)
    want = orc.expert_union_plan_bytes(entries, R, K)
    assert np.array_equal(un.plan.cpu().numpy(), want)                      # header, the entries, and the unused entries as the builder leaves them
    assert len(entries) < R * K or R < 3                                    # from three rows on the rows do share experts
    for name in FIELDS:
        got = getattr(un, name).cpu().numpy()
        for r in range(R):
            assert np.array_equal(bits(got[r]) if got.dtype == np.float32 else got[r],
                                  bits(rows[r][name][0]) if got.dtype == np.float32 else rows[r][name][0]), (name, r)


@pytest.mark.parametrize("H,I,E,K,R,same", [
    (512, 256, 16, 3, 1, False),       # one row, top-3: the routes view is 12 bytes (a single row slice needs no 16-byte pitch)
    (1024, 512, 16, 8, 8, True),       # every row names the same eight experts in its own order: eight holders per entry
    (1024, 512, 16, 4, 7, True)])      # seven holders: the last sweep of an entry serves three rows
def test_union_rows_small_shapes_and_full_entries(strix, H, I, E, K, R, same):
    rng = np.random.default_rng(3 * H + R)
    gate, up, down = make_layer(rng, H, I, E)
    pool = rng.permutation(E)[:K]
    ids = np.stack([rng.permutation(pool) if same else rng.permutation(E)[:K] for _ in range(R)]).astype(np.uint32)
    rows, un, _ = run_paths(strix, rng, H, I, E, K, R, orc.Q4_K, ids, gate, up, down)
    assert int(un.status.item()) == 0
    entries = orc.expert_union_build(ids, R, K, E)
    assert np.array_equal(un.plan.cpu().numpy(), orc.expert_union_plan_bytes(entries, R, K))
    if same:
        assert len(entries) == K and all(sum(s != orc.UNION_NO_SLOT for s in slots) == R for _, slots in entries)
    for name in FIELDS:
        got = getattr(un, name).cpu().numpy()
        for r in range(R):
            a, b = got[r], rows[r][name][0]
            assert np.array_equal(bits(a) if a.dtype == np.float32 else a, bits(b) if b.dtype == np.float32 else b), (name, r)


def test_union_rows_against_the_oracle(strix):
    H, I, E, K, R = 1024, 512, 16, 4, 6
    rng = np.random.default_rng(77)
    gate, up, down = make_layer(rng, H, I, E)
    ids = np.stack([rng.permutation(E)[:K] for _ in range(R)]).astype(np.uint32)
    _, un, x = run_paths(strix, rng, H, I, E, K, R, orc.Q4_K, ids, gate, up, down, kind=torch.bfloat16)
    c, d, s, _ = orc.quantize_a8(x.to(torch.float32).numpy())
    ref = orc.routed_experts(H, I, K, gate, up, down, orc.Q4_K, c, d, s, ids)
    out = un.intermediates.cpu().numpy()
    assert np.array_equal(bits(out[:, :, 0]), bits(ref.h.reshape(R, K, I))) and np.array_equal(bits(out[:, :, 1]), bits(ref.up.reshape(R, K, I)))
    assert np.array_equal(un.h_codes.cpu().numpy().reshape(R * K, I), ref.h_codes)
    assert np.array_equal(bits(un.h_deltas.cpu().numpy().reshape(R * K, I // 32)), bits(ref.h_deltas))
    assert np.array_equal(bits(un.rawdots.cpu().numpy()), bits(ref.rawdots.reshape(R, K, H)))


def test_union_refuses_a_repeated_expert_and_an_id_out_of_range(strix):
    H, I, E, K, R = 1024, 512, 16, 4, 2
    rng = np.random.default_rng(5)
    gate, up, down = make_layer(rng, H, I, E)
    for ids in (np.array([[3, 3, 1, 2], [4, 5, 6, 7]], np.int32), np.array([[0, 1, 2, 3], [4, E, 6, 7]], np.int32)):
        p = strix.A8Decode(H, I, E, K, dev(gate), dev(up), dev(down), rows=R, input_dtype=torch.float32)
        p.input.copy_(torch.from_numpy(rng.standard_normal((R, H)).astype(np.float32)))
        p.routes.copy_(torch.from_numpy(ids))
        p.intermediates.fill_(-7.0)
        p.enqueue_probe_union()
        torch.cuda.synchronize()
        assert int(p.status.item()) == strix.STATUS_INVALID_ROUTE           # exactly the invalid-route bit (hip_moe_a8_union_tests.hip:155)
        plan = p.plan.cpu().numpy()
        assert plan[:16].view(np.uint32).tolist() == [0, R, K, 0]           # no entry is swept
        assert np.all(p.intermediates.cpu().numpy() == -7.0)
    # the same routes in two rows are admitted (tests/moe_expert_union_tests.cpp:64)
    p = strix.A8Decode(H, I, E, K, dev(gate), dev(up), dev(down), rows=R, input_dtype=torch.float32)
    p.input.copy_(torch.from_numpy(rng.standard_normal((R, H)).astype(np.float32)))
    p.routes.copy_(torch.tensor([[3, 4, 5, 6], [3, 4, 5, 6]], dtype=torch.int32))
    p.enqueue_probe_union()
    torch.cuda.synchronize()
    assert int(p.status.item()) == 0 and p.plan.cpu().numpy()[:4].view(np.uint32)[0] == 4
