"""The strided per-row views (the reference's Rows / Strided<T>, include/strix/cuda/qwen_moe.hpp:34-37,55-76, stages :96-110) and
the host executor's job form (Job / Assignment / RowA8, src/cpu/core/routed_expert.hpp:41-61) on the GPU, bit for bit against
the CPU oracle and, for the job form, against the compiled reference's reference_run where it was built."""
import ctypes as C

import numpy as np
import pytest
import torch

import orc
from test_gpu_parity import bits, dev, make_layer
from test_gpu_a8_contract import make_down

pytestmark = pytest.mark.gpu


def pad16(n):
    return (n + 15) // 16 * 16


class RowBlocks:
    """Every per-row view inside one block of bytes per row (an array of row records: the layout of a caller whose planner
    carves one workspace extent per row), so that every view has the same, non-dense stride."""

    FIELDS = ("input", "routes", "route_weights", "codes", "deltas", "sums", "status", "intermediates", "accumulation", "down_codes",
              "down_deltas", "down_sums", "rawdots", "output")

    def __init__(self, strix, T, H, I, K, E, in_dtype, out_dtype, spare=48):
        isz = torch.empty(0, dtype=in_dtype).element_size()
        osz = torch.empty(0, dtype=out_dtype).element_size()
        sizes = dict(input=H * isz, routes=4 * K, route_weights=4 * K, codes=H, deltas=H // 8, sums=H // 8, status=4, intermediates=8 * K * I,
                     accumulation=4 * H, down_codes=K * I, down_deltas=K * I // 8, down_sums=K * I // 8, rawdots=4 * K * H, output=H * osz)
        self.at, off = {}, 0
        for f in self.FIELDS:
            self.at[f] = off
            off += pad16(sizes[f]) + 16
        self.stride = pad16(off + spare)
        self.sizes, self.T = sizes, T
        self.buf = torch.full((T, self.stride), 0x5A, dtype=torch.uint8, device="cuda")
        self.plan = torch.zeros(strix.lib().mi355_moe_plan_words(E, T, K), dtype=torch.int32, device="cuda")
        self.job = torch.zeros(1, dtype=torch.int32, device="cuda")
        v = strix.MoeRowsStrided()
        for f in self.FIELDS:
            setattr(v, f, strix.Strided(self.buf.data_ptr() + self.at[f], self.stride))
        v.plan, v.job_status = self.plan.data_ptr(), self.job.data_ptr()
        v.input_kind, v.output_kind = strix.input_kind(torch.empty(0, dtype=in_dtype)), strix.input_kind(torch.empty(0, dtype=out_dtype))
        self.view = v

    def put(self, field, rows):
        """rows: a [T, ...] tensor; its bytes go to the field of every row."""
        raw = rows.contiguous().view(torch.uint8).reshape(self.T, -1).cuda()
        self.buf[:, self.at[field]: self.at[field] + raw.shape[1]] = raw

    def get(self, field, dtype, shape):
        raw = self.buf[:, self.at[field]: self.at[field] + self.sizes[field]].contiguous().cpu()
        return raw.view(dtype).reshape((self.T,) + shape).numpy() if dtype != torch.bfloat16 else raw.view(dtype).reshape((self.T,) + shape)


def weights_of(strix, H, I, E, K, gate, up, down, gate_type, down_type):
    w = strix.MoeWeights()
    w.hidden, w.ffn, w.experts, w.top_k, w.gate_type, w.down_type = H, I, E, K, gate_type, down_type
    w.gate, w.up, w.down = gate.data_ptr(), up.data_ptr(), down.data_ptr()
    w.exp_kind, w.swiglu_limit = strix.EXP_GFX1151, float("inf")
    return w


@pytest.mark.parametrize("gate_type,down_type,H,I,E,K,T,in_kind,out_kind", [
    (orc.Q4_K, orc.Q4_K, 2048, 768, 128, 8, 8, torch.bfloat16, torch.bfloat16),       # config 3: 64 assignments, the 64-row sweeps
    (orc.Q4_K, orc.Q4_K, 1024, 512, 16, 4, 3, torch.bfloat16, torch.float32),         # 12 assignments, the 16-row sweeps
    (orc.Q5_K, orc.Q8_0, 1024, 512, 16, 4, 40, torch.float16, torch.bfloat16),        # the reference twin's own formats, shared sweeps
    (orc.Q4_K, orc.Q5_1, 2560, 640, 64, 10, 16, torch.bfloat16, torch.bfloat16),      # the twin's fixed geometry but for the expert count
    (orc.Q4_K, orc.Q6_K, 512, 768, 6, 3, 5, torch.float32, torch.float32),
    (orc.Q4_K, orc.Q4_K, 1024, 1024, 1, 1, 6, torch.bfloat16, torch.bfloat16),        # a dense matrix through strided views (matrix-core sweep)
    (orc.Q4_K, orc.Q4_K, 512, 512, 4, 2, 40, torch.bfloat16, torch.float32)])         # 20 rows per expert: items of up to 128 rows on the matrix-core sweep
def test_strided_rows_every_stage(strix, gate_type, down_type, H, I, E, K, T, in_kind, out_kind):
    rng = np.random.default_rng(H + I + 3 * T + down_type)
    if I % 256 == 0:
        gate, up, _ = make_layer(rng, H, I, E)
    else:
        gate = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((E, I, H)) * 0.05).astype(np.float32))
        up = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((E, I, H)) * 0.05).astype(np.float32))
    if gate_type == orc.Q5_K:
        gate, up = orc.random_q5_k(rng, (E, I), H), orc.random_q5_k(rng, (E, I), H)
    down = make_down(rng, down_type, E, H, I)
    x_t = torch.from_numpy(rng.standard_normal((T, H)).astype(np.float32)).to(in_kind)
    x32 = x_t.to(torch.float32).numpy()
    ids = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.uint32)
    wts = rng.random((T, K)).astype(np.float32)
    wts /= wts.sum(1, keepdims=True)
    g_d, u_d, d_d = dev(gate), dev(up), dev(down)
    w = weights_of(strix, H, I, E, K, g_d, u_d, d_d, gate_type, down_type)
    rb = RowBlocks(strix, T, H, I, K, E, in_kind, out_kind)
    rb.put("input", x_t)
    rb.put("routes", torch.from_numpy(ids.astype(np.int32)))
    rb.put("route_weights", torch.from_numpy(wts))
    record = torch.zeros(2, dtype=torch.int32, device="cuda")
    L = strix.lib()
    before = rb.buf.clone()
    st = None
    assert L.mi355_moe_strided_enqueue_prologue(C.byref(w), C.byref(rb.view), T, H, st) == 0, L.mi355_last_error()
    assert L.mi355_moe_strided_enqueue_csr(C.byref(w), C.byref(rb.view), T, st) == 0, L.mi355_last_error()
    assert L.mi355_moe_strided_enqueue_project(C.byref(w), C.byref(rb.view), T, st) == 0, L.mi355_last_error()
    assert L.mi355_moe_strided_enqueue_down(C.byref(w), C.byref(rb.view), T, st) == 0, L.mi355_last_error()
    assert L.mi355_moe_strided_enqueue_merge(C.byref(w), C.byref(rb.view), T, st) == 0, L.mi355_last_error()
    assert L.mi355_moe_strided_enqueue_commit(C.byref(w), C.byref(rb.view), T, record.data_ptr(), 2, st) == 0, L.mi355_last_error()
    torch.cuda.synchronize()
    c, d, s, _ = orc.quantize_a8(x32, tiny_rule=False)
    assert np.array_equal(rb.get("codes", torch.int8, (H,)), c) and np.array_equal(bits(rb.get("deltas", torch.float32, (H // 32,))), bits(d))
    assert np.array_equal(rb.get("sums", torch.int32, (H // 32,)), s)
    assert np.all(rb.get("status", torch.int32, (1,)) == 0) and int(rb.job.item()) == 0 and record.tolist() == [0, 0]
    ref = orc.routed_experts(H, I, K, gate, up, down, down_type, c, d, s, ids, gate_type=gate_type)
    inter = rb.get("intermediates", torch.float32, (K, 2, I))
    assert np.array_equal(bits(inter[:, :, 0]), bits(ref.h.reshape(T, K, I))) and np.array_equal(bits(inter[:, :, 1]), bits(ref.up.reshape(T, K, I)))
    assert np.array_equal(rb.get("down_codes", torch.int8, (K, I)), ref.h_codes.reshape(T, K, I))
    assert np.array_equal(bits(rb.get("down_deltas", torch.float32, (K, I // 32))), bits(ref.h_deltas.reshape(T, K, -1)))
    assert np.array_equal(rb.get("down_sums", torch.int32, (K, I // 32)), ref.h_sums.reshape(T, K, -1))
    raw = rb.get("rawdots", torch.float32, (K, H))
    assert np.array_equal(bits(raw), bits(ref.rawdots))
    want = orc.combine(0, wts, ids, ref.rawdots)
    assert np.array_equal(bits(rb.get("accumulation", torch.float32, (H,))), bits(want))
    if out_kind == torch.float32:
        assert np.array_equal(bits(rb.get("output", torch.float32, (H,))), bits(want))
    else:
        assert torch.equal(rb.get("output", torch.bfloat16, (H,)), torch.from_numpy(want).to(torch.bfloat16))
    # nothing outside the fields was written: the gaps between them and the spare tail of every row block still hold the fill
    mask = torch.ones(rb.stride, dtype=torch.bool)
    for f in rb.FIELDS:
        mask[rb.at[f]: rb.at[f] + rb.sizes[f]] = False
    assert torch.equal(rb.buf[:, mask.cuda()], before[:, mask.cuda()])
    # the single call gives the same bytes
    rb2 = RowBlocks(strix, T, H, I, K, E, in_kind, out_kind, spare=16)
    rb2.put("input", x_t)
    rb2.put("routes", torch.from_numpy(ids.astype(np.int32)))
    rb2.put("route_weights", torch.from_numpy(wts))
    assert L.mi355_moe_strided_enqueue(C.byref(w), C.byref(rb2.view), T, H, record.data_ptr(), 2, st) == 0, L.mi355_last_error()
    torch.cuda.synchronize()
    for f in ("rawdots", "accumulation", "output", "down_codes"):
        a0, n = rb.at[f], rb.sizes[f]
        b0 = rb2.at[f]
        assert torch.equal(rb.buf[:, a0: a0 + n], rb2.buf[:, b0: b0 + n]), f


def test_strided_rows_fail_closed_and_first_error_record(strix):
    """An invalid route fails the whole job: its row carries status 1 and no image, the job word is set by the plan stage, no row
    is merged or committed, and the record names the first failed row's bits (src/cuda/models/qwen/qwen_moe.cu:287-340)."""
    H, I, E, K, T = 1024, 512, 16, 4, 6
    rng = np.random.default_rng(11)
    gate, up, down = make_layer(rng, H, I, E)
    g_d, u_d, d_d = dev(gate), dev(up), dev(down)
    w = weights_of(strix, H, I, E, K, g_d, u_d, d_d, orc.Q4_K, orc.Q4_K)
    rb = RowBlocks(strix, T, H, I, K, E, torch.bfloat16, torch.bfloat16)
    x = rng.standard_normal((T, H)).astype(np.float32)
    ids = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.int32)
    ids[3, 2] = E + 5
    wts = np.full((T, K), 0.25, np.float32)
    wts[4, 1] = np.inf                              # a non-finite route weight is an invalid route too
    rb.put("input", torch.from_numpy(x).to(torch.bfloat16))
    rb.put("routes", torch.from_numpy(ids))
    rb.put("route_weights", torch.from_numpy(wts))
    record = torch.zeros(2, dtype=torch.int32, device="cuda")
    L = strix.lib()
    assert L.mi355_moe_strided_enqueue(C.byref(w), C.byref(rb.view), T, H, record.data_ptr(), 2, None) == 0, L.mi355_last_error()
    torch.cuda.synchronize()
    status = rb.get("status", torch.int32, (1,))[:, 0]
    assert status.tolist() == [0, 0, 0, 1, 1, 0] and int(rb.job.item()) == 1 and record.tolist() == [2, 1]
    assert np.all(rb.get("accumulation", torch.float32, (H,)) == 0.0)             # cleared by the prologue, never merged
    assert np.all(rb.get("output", torch.int16, (H,)) == 0x5A5A)                  # nothing committed
    assert np.all(rb.get("codes", torch.int8, (H,))[3] == 0x5A)                    # the failed row was not quantised
    # a second failing step leaves the first record
    assert L.mi355_moe_strided_enqueue(C.byref(w), C.byref(rb.view), T, H, record.data_ptr(), 7, None) == 0
    assert record.tolist() == [2, 1]
    # non-finite input: bit 2, taken as 0
    ids[3, 2] = 1
    wts[4, 1] = 0.25
    x[2, 9] = np.nan
    rb.put("input", torch.from_numpy(x).to(torch.bfloat16))
    rb.put("routes", torch.from_numpy(ids))
    rb.put("route_weights", torch.from_numpy(wts))
    record.zero_()
    assert L.mi355_moe_strided_enqueue(C.byref(w), C.byref(rb.view), T, H, record.data_ptr(), 2, None) == 0
    status = rb.get("status", torch.int32, (1,))[:, 0]
    assert status.tolist() == [0, 0, 2, 0, 0, 0] and record.tolist() == [2, 2]


def test_strided_rows_admission(strix):
    H, I, E, K, T = 1024, 512, 16, 4, 2
    rng = np.random.default_rng(12)
    gate, up, down = make_layer(rng, H, I, E)
    g_d, u_d, d_d = dev(gate), dev(up), dev(down)
    w = weights_of(strix, H, I, E, K, g_d, u_d, d_d, orc.Q4_K, orc.Q4_K)
    rb = RowBlocks(strix, T, H, I, K, E, torch.bfloat16, torch.bfloat16)
    L = strix.lib()
    before = rb.buf.clone()
    v = rb.view
    keep = v.rawdots.stride
    v.rawdots.stride = 4 * K * H - 16                       # shorter than a row's extent
    assert L.mi355_moe_strided_enqueue(C.byref(w), C.byref(v), T, H, None, 2, None) == -1
    v.rawdots.stride = keep
    v.codes.base += 8                                       # misaligned
    assert L.mi355_moe_strided_enqueue(C.byref(w), C.byref(v), T, H, None, 2, None) == -1
    v.codes.base -= 8
    v.output_kind = 1                                       # fp16 output is not a form
    assert L.mi355_moe_strided_enqueue(C.byref(w), C.byref(v), T, H, None, 2, None) == -1
    v.output_kind = 2
    assert L.mi355_moe_strided_enqueue_prologue(C.byref(w), C.byref(v), T, rb.stride, None) == -1      # clear_words beyond the row
    torch.cuda.synchronize()
    assert torch.equal(rb.buf, before)


# ------------------------------------------------------------------------------------------------------- job form
def make_job(strix, rng, H, I, E, T, n, gate_type, down_type, gate, up, down, stride_pad=64, slots=4):
    x = rng.standard_normal((T, H)).astype(np.float32)
    c, d, s, _ = orc.quantize_a8(x)
    # the A8 image of every row in an allocation of its own
    imgs = [(dev(c[t]), dev(d[t]), dev(s[t])) for t in range(T)]
    table = (strix.RowA8 * T)(*[strix.RowA8(a.data_ptr(), b.data_ptr(), cc.data_ptr()) for a, b, cc in imgs])
    table_d = torch.frombuffer(bytearray(bytes(table)), dtype=torch.uint8).cuda()
    # assignments in no particular order: rows have different numbers of slots, experts repeat
    pairs = [(t, k) for t in range(T) for k in range(slots)]
    rng.shuffle(pairs)
    pairs = pairs[:n]
    asg = np.array([[t, k, rng.integers(E)] for t, k in pairs], np.uint32)
    stride = slots * H + stride_pad
    raw = torch.full((T, stride), -7.0, device="cuda")
    status = torch.zeros(T, dtype=torch.int32, device="cuda")
    job = strix.ExpertJob()
    job.weights = strix.LayerWeights(gate.data_ptr(), up.data_ptr(), down.data_ptr(), int(gate_type == orc.Q5_K), int(down_type == orc.Q8_0), H, I)
    asg_d = dev(asg)
    job.rows, job.assignments, job.count = table_d.data_ptr(), asg_d.data_ptr(), len(asg)
    job.rawdots, job.rawdot_row_stride, job.status = raw.data_ptr(), stride, status.data_ptr()
    keep = (imgs, table_d, asg_d)
    return job, keep, (c, d, s), asg, raw, status, stride


@pytest.mark.parametrize("gate_type,down_type,H,I,E,T,n", [
    (orc.Q4_K, orc.Q8_0, 512, 256, 6, 5, 15),              # the shape of the compiled reference's own whole-job check
    (orc.Q4_K, orc.Q5_1, 512, 256, 6, 5, 15),
    (orc.Q5_K, orc.Q8_0, 512, 384, 6, 5, 9),               # ffn a multiple of 128 only
    (orc.Q4_K, orc.Q8_0, 2048, 768, 128, 8, 30),           # 30 assignments: the two-slot 16-row sweep
    (orc.Q5_K, orc.Q5_1, 2048, 768, 128, 8, 32),
    (orc.Q4_K, orc.Q5_1, 1024, 640, 16, 24, 90)])          # 90 assignments: the 64-row sweep
def test_executor_job_form(strix, gate_type, down_type, H, I, E, T, n):
    rng = np.random.default_rng(H + I + n + down_type)
    if gate_type == orc.Q5_K:
        gate, up = orc.random_q5_k(rng, (E, I), H), orc.random_q5_k(rng, (E, I), H)
    else:
        gate = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((E, I, H)) * 0.05).astype(np.float32))
        up = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((E, I, H)) * 0.05).astype(np.float32))
    down = make_down(rng, down_type, E, H, I)
    g_d, u_d, d_d = dev(gate), dev(up), dev(down)
    job, keep, (c, d, s), asg, raw, status, stride = make_job(strix, rng, H, I, E, T, n, gate_type, down_type, g_d, u_d, d_d)
    ex = strix.Executor(max_assignments=128, max_ffn=1024)
    ex.run(job)
    torch.cuda.synchronize()
    # the oracle, one assignment at a time (a one-slot row per assignment)
    rows = asg[:, 0]
    ref = orc.routed_experts(H, I, 1, gate, up, down, down_type, c[rows], d[rows], s[rows], asg[:, 2:3].copy(), gate_type=gate_type)
    got = raw.cpu().numpy()
    want = np.full_like(got, -7.0)
    for a, (t, k, _) in enumerate(asg):
        want[t, k * H: (k + 1) * H] = ref.rawdots[a, 0]
    assert np.array_equal(bits(got), bits(want))               # every assignment's outputs, and nothing else, was written
    assert torch.all(status == 0)
    R = orc.ref()
    if R:
        raw_ref = np.full((raw.shape[0], stride), -7.0, np.float32)
        st_ref = np.zeros(raw.shape[0], np.uint32)
        rc = R.ref_routed_expert_run_fmt(H, I, gate.ctypes.data_as(orc.u8p), up.ctypes.data_as(orc.u8p), down.ctypes.data_as(orc.u8p),
                                         int(down_type == orc.Q5_1) + 2 * int(gate_type == orc.Q5_K), c.ctypes.data_as(orc.i8p), d.ctypes.data_as(orc.f32p),
                                         s.ctypes.data_as(orc.i32p), raw.shape[0], asg.ctypes.data_as(orc.u32p), len(asg), raw_ref.ctypes.data_as(orc.f32p),
                                         C.c_uint64(stride), st_ref.ctypes.data_as(orc.u32p), 0, 0)
        assert rc == 0, R.ref_last_error()
        assert np.array_equal(bits(got), bits(raw_ref))
        print("device job == compiled reference_run, %d assignments" % len(asg))
    ex.close()


def test_executor_job_nonfinite_fails_closed_and_limits(strix):
    H, I, E, T, n = 512, 256, 6, 4, 10
    rng = np.random.default_rng(5)
    gate = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((E, I, H)) * 0.05).astype(np.float32))
    up = orc.quantize_rows(orc.Q4_K, (rng.standard_normal((E, I, H)) * 0.05).astype(np.float32))
    down = make_down(rng, orc.Q8_0, E, H, I)
    g_d, u_d, d_d = dev(gate), dev(up), dev(down)
    job, keep, (c, d, s), asg, raw, status, stride = make_job(strix, rng, H, I, E, T, n, orc.Q4_K, orc.Q8_0, g_d, u_d, d_d)
    bad_row = int(asg[3, 0])
    keep[0][bad_row][1][2] = float("inf")                        # a delta of that row: its gate / up rows are not finite
    ex = strix.Executor(max_assignments=16, max_ffn=256)
    ex.run(job)
    torch.cuda.synchronize()
    want = [1 if t == bad_row else 0 for t in range(T)]
    assert status.tolist() == want                               # kNonfinite = 1 in the row's word
    assert torch.all(raw == -7.0)                                # a failed job computes no down row
    # the next job on the same executor starts clean
    keep[0][bad_row][1][2] = float(d[bad_row][2])
    status.zero_()
    ex.run(job)
    assert torch.all(status == 0) and not torch.all(raw == -7.0)
    # limits are refused before any launch
    L = strix.lib()
    job.count = 17
    assert L.mi355_executor_run(ex.handle, C.byref(job), None) == -1 and b"larger than the executor" in L.mi355_last_error()
    job.count = 0
    assert L.mi355_executor_run(ex.handle, C.byref(job), None) == 0          # an empty job is nothing
    assert not L.mi355_executor_create(0, 256, 0) and not L.mi355_executor_create(16, 100, 0)
    ex.close()


# ---------------------------------------------------------------------------------- the fp16 prefill over strided rows
def _bf16_round(a):
    b = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    return (((b + 0x7fff + ((b >> 16) & 1)) & 0xffff0000).astype(np.uint32)).view(np.float32)


@pytest.mark.parametrize("gate_type,down_type,H,I,E,K,T", [
    (orc.Q4_K, orc.Q4_K, 1024, 512, 8, 2, 70),          # the register-operand kernels (one down pass)
    (orc.Q8_0, orc.Q8_0, 512, 256, 4, 2, 33),           # the loader / multiplier kernels (two down passes: the rounding belongs to the second)
    (orc.Q4_K, orc.Q4_K, 2048, 768, 16, 4, 9)])
def test_prefill_rows_f16_strided_views(strix, gate_type, down_type, H, I, E, K, T):
    """mi355_moe_enqueue_prefill_rows_f16 (known_rows::PrefillRows / enqueue_prefill with the fp16 form,
    include/strix/hip_moe_q4k_a8_known_rows.hpp:75-111): every view strided inside one record per row. The unweighted outputs are
    bit for bit those of the dense entry point (the same kernels behind another view), with rawdots_bf16 their bfloat16 rounding;
    the prologue zeroes the clear words, overwrites the status words and flags a bad route or route weight; the caller's merge
    over the same strided views gives the dense entry's combined rows."""
    rng = np.random.default_rng(H + T)
    if gate_type == orc.Q8_0:
        gate, up = (orc.quantize_rows(orc.Q8_0, (rng.standard_normal((E, I, H)) * 0.05).astype(np.float32)) for _ in range(2))
        down = orc.quantize_rows(orc.Q8_0, (rng.standard_normal((E, H, I)) * 0.05).astype(np.float32))
    else:
        gate, up, down = make_layer(rng, H, I, E)
    x = rng.standard_normal((T, H)).astype(np.float16)
    ids = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.int32)
    wts = rng.random((T, K)).astype(np.float32)
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T, prefill_f16=True, gate_type=gate_type, down_type=down_type)
    dense_raw = layer.run_prefill_f16(dev(x), dev(ids), dev(wts), combine=strix.COMBINE_NONE).cpu().numpy().copy()
    assert int(layer.status.sum()) == 0
    dense_out = layer.run_prefill_f16(dev(x), dev(ids), dev(wts)).cpu().numpy().copy()

    sizes = dict(input=2 * H, routes=4 * K, route_weights=4 * K, status=4, clear=4 * H, rawdots=4 * K * H)
    at, off = {}, 0
    for f, n in sizes.items():
        at[f] = off
        off += pad16(n) + 32
    stride = pad16(off + 16)
    for bf16 in (False, True):
        buf = torch.full((T, stride), 0x5A, dtype=torch.uint8, device="cuda")
        put = lambda f, a: buf.__setitem__((slice(None), slice(at[f], at[f] + sizes[f])), torch.from_numpy(np.ascontiguousarray(a)).view(torch.uint8).reshape(T, -1).cuda())
        get = lambda f, dt, shape: buf[:, at[f]: at[f] + sizes[f]].contiguous().cpu().numpy().view(dt).reshape((T,) + shape)
        put("input", x); put("routes", ids); put("route_weights", wts)
        v = strix.PrefillRows()
        for f in sizes:
            setattr(v, f, strix.Strided(buf.data_ptr() + at[f], stride))
        v.rawdots_bf16 = 1 if bf16 else 0
        layer.run_prefill_rows_f16(v, T, clear_words=H - 7)
        torch.cuda.synchronize()
        raw = get("rawdots", np.float32, (K, H))
        assert np.array_equal(bits(raw), bits(_bf16_round(dense_raw) if bf16 else dense_raw)), bf16
        clear = get("clear", np.uint32, (H,))
        assert np.all(clear[:, :H - 7] == 0) and np.all(clear[:, H - 7:] == 0x5A5A5A5A)
        assert np.all(get("status", np.uint32, (1,)) == 0) and int(layer.job_status[0]) == 0
        assert np.all(buf[:, at["status"] + 4: at["clear"]].cpu().numpy() == 0x5A)          # nothing past a field's extent
    # the caller's merge over the same views (fp32 rawdots): the dense entry's combined rows
    buf = torch.full((T, stride), 0x5A, dtype=torch.uint8, device="cuda")
    put = lambda f, a: buf.__setitem__((slice(None), slice(at[f], at[f] + sizes[f])), torch.from_numpy(np.ascontiguousarray(a)).view(torch.uint8).reshape(T, -1).cuda())
    put("input", x); put("routes", ids); put("route_weights", wts)
    v = strix.PrefillRows()
    for f in sizes:
        setattr(v, f, strix.Strided(buf.data_ptr() + at[f], stride))
    layer.run_prefill_rows_f16(v, T)
    merged = strix.combine(strix.COMBINE_FMA_SLOT, torch.from_numpy(dense_raw).cuda(), dev(wts), torch.zeros((T, H), dtype=torch.float32, device="cuda"))
    assert np.array_equal(bits(merged.cpu().numpy()), bits(dense_out))
    # a route that names no expert and a non-finite route weight: bit 1 in those rows, overwritten stale words elsewhere
    bad_ids, bad_w = ids.copy(), wts.copy()
    bad_ids[1, 0] = E
    bad_w[T - 1, K - 1] = np.inf
    put("routes", bad_ids); put("route_weights", bad_w)
    layer.run_prefill_rows_f16(v, T)
    torch.cuda.synchronize()
    status = buf[:, at["status"]: at["status"] + 4].contiguous().cpu().numpy().view(np.uint32)[:, 0]
    want = np.zeros(T, np.uint32); want[1] = 1; want[T - 1] = 1
    assert np.array_equal(status, want)
    with pytest.raises(strix.StrixError, match="clear_words"):
        layer.run_prefill_rows_f16(v, T, clear_words=stride)
