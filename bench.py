#!/usr/bin/env python3
"""Benchmark of the quantized weight-product path on one MI355X.

A step is one pass of the headline workload, BASELINE config 3: one MoE decode layer (hidden 2048, 128 experts, softmax
router top-8, expert intermediate 768, Q4_K gate/up/down, 8 fp16 tokens) = router + A8 prologue + expert plan + gate/up/
SwiGLU/re-quantise + down + ordered combine. Inputs are resident in HBM before the timed region. To keep the experts out
of the 256 MB last-level cache between steps, the steps rotate over several independent layers (distinct weights and
tokens), as consecutive layers of a model do.

Prints ONE JSON line. `value` = microseconds per layer (lower is better). `roofline` prices the dominant kernel (the layer's
front launch: early routes, A8 prologue, the exact router and the gate/up projection) by its algorithmic bytes against the
8 TB/s HBM peak, from HIP events recorded around that launch on its own stream inside this run. `prefill` is the metric's second figure: BASELINE config 4 (4096 rows) on the matrix cores, TFLOP/s against
the fp16 MFMA peak. `cpu_baseline` times the CPU oracle (a port of the reference's CPU path) on the same layer, with the
compiled reference's own Executor beside it where that library was built, the host CPU model and its read-bandwidth ceiling."""
import argparse
import ctypes as C
import json
import os
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBPS = 8000.0     # MI355X published HBM3E peak
MFMA_F16_PEAK_FLOPS = 2.5e15     # MI355X published dense fp16 MFMA peak
# HBM bytes per launch of the layer's front kernel on the default workload, from two rocprofv3 --pmc passes (FETCH_SIZE scaled
# x2.000, WRITE_SIZE x1.000 by a 256 MiB device copy in the same runs): profiles/layer_front_kernel_config3_moe_decode_T8.txt
FRONT_TRAFFIC_BYTES_DEFAULT = 94_804_992
FRONT_TRAFFIC_SOURCE = "profiles/layer_front_kernel_config3_moe_decode_T8.txt (a constant from that profile, not measured in this run)"
Q4K_ROW = lambda k: k // 256 * 144


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--tokens", type=int, default=8)
    ap.add_argument("--layers", type=int, default=5, help="independent layers rotated through (cold-cache working set); at most --warmup of them, so that none is first run inside the timed steps")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-prefill", action="store_true", help="skip the config-4 prefill leg")
    ap.add_argument("--extra", action="store_true",
                    help="also time BASELINE configs 1, 2, 4 and 5 (reported under 'extra'; the headline value stays config 3)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy 4 times (a kernel of known HBM traffic, for scaling rocprof FETCH_SIZE / WRITE_SIZE)")
    return ap.parse_args()


class Config3:
    H, I, E, K = 2048, 768, 128, 8

    def __init__(self, strix, torch, layers, tokens, seed=3):
        self.strix, self.torch, self.T = strix, torch, tokens
        g = torch.Generator(device="cuda").manual_seed(seed)
        H, I, E, K = self.H, self.I, self.E, self.K
        self.layers = []
        for _ in range(layers):
            q = lambda shape: strix.quantize_weight_rows(strix.TYPE_Q4_K, torch.randn(shape, generator=g, device="cuda") * 0.02)
            gate, up, down = q((E, I, H)), q((E, I, H)), q((E, H, I))
            wr = torch.randn((E, H), generator=g, device="cuda") * 0.02
            x = torch.randn((tokens, H), generator=g, device="cuda").to(torch.float16)
            layer = strix.MoeLayer(H, I, E, K, gate, up, down, tokens)
            self.layers.append((layer, wr, x))
        torch.cuda.synchronize()

    def step(self, i):
        layer, wr, x = self.layers[i % len(self.layers)]
        layer.run_layer(x, wr)

    def staged_step(self, i, events):
        """Same work, one entry point per stage, with an event pair around each stage on the launch stream."""
        torch, strix = self.torch, self.strix
        layer, wr, x = self.layers[i % len(self.layers)]
        marks = [torch.cuda.Event(enable_timing=True) for _ in range(7)]
        marks[0].record()
        ids, wts, _ = strix.route(x, wr, self.K)
        marks[1].record()
        for n, name in enumerate(("prologue", "csr", "project", "down", "merge")):
            layer.stage(name, x, ids, wts)
            marks[2 + n].record()
        events.append(marks)
        return ids

    def project_launch_us(self, reps):
        """Mean duration of the projection launch: every layer is brought to the state just before it (router, prologue,
        plan), then the projection of all layers is enqueued back to back between ONE pair of events on the launch stream
        (the weights of the rotation do not fit the last-level cache, so every launch streams from HBM)."""
        torch, strix = self.torch, self.strix
        total = 0.0
        for _ in range(reps):
            staged = []
            for layer, wr, x in self.layers:
                ids, wts, _ = strix.route(x, wr, self.K)
                layer.stage("prologue", x, ids, wts)
                layer.stage("csr", x, ids, wts)
                staged.append((layer, x, ids, wts))
            t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0.record()
            for layer, x, ids, wts in staged:
                layer.stage("project", x, ids, wts)
            t1.record()
            torch.cuda.synchronize()
            total += t0.elapsed_time(t1) * 1e3 / len(staged)
            for layer, x, ids, wts in staged:       # leave every layer's buffers complete
                layer.stage("down", x, ids, wts)
                layer.stage("merge", x, ids, wts)
        return total / reps

    def halves_launch_us(self, reps):
        """Mean durations of the layer's two launches on the timed path (mi355_moe_enqueue_layer_front / _back: the kernels the
        whole call enqueues): the front launches of all rotating layers back to back between ONE pair of events on the launch
        stream, then the back launches likewise (the pairs also span the gaps between the launches, about 1.5 us each)."""
        torch = self.torch
        front = back = 0.0
        for _ in range(reps):
            e = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
            e[0].record()
            for layer, wr, x in self.layers:
                layer.run_layer(x, wr, half="front")
            e[1].record()
            e[2].record()
            for layer, wr, x in self.layers:
                layer.run_layer(x, wr, half="back")
            e[3].record()
            torch.cuda.synchronize()
            front += e[0].elapsed_time(e[1]) * 1e3 / len(self.layers)
            back += e[2].elapsed_time(e[3]) * 1e3 / len(self.layers)
        return front / reps, back / reps

    def front_bytes(self, u):
        # the front launch: router weight and the rows, gate + up rows of the touched experts, the A8 image written and read, the h image written
        return self.E * self.H * 4 + self.T * self.H * 2 + self.project_bytes(u)

    def distinct_experts(self):
        out = []
        for layer, wr, x in self.layers:
            ids, _, _ = self.strix.route(x, wr, self.K)
            out.append(int(self.torch.unique(ids).numel()))
        return out

    def layer_bytes(self, u):
        return u * 3 * self.I * Q4K_ROW(self.H) + self.E * self.H * 4 + self.T * (self.H * 2 + self.H * 4)

    def project_bytes(self, u):
        # gate + up rows of the touched experts, the A8 image read and the h image written
        return u * 2 * self.I * Q4K_ROW(self.H) + self.T * self.H * 1.25 + self.T * self.K * self.I * 1.25


def device_q4k(torch, gen, rows_shape, width, d_bits=0x13):
    """Random Q4_K blocks with finite, moderate fp16 d / dmin (every other bit random) - no fp32 staging tensor needed.
    d_bits = 0x03 keeps d below 2^-11 (weights of a few hundredths), so that a 4096-wide product stays far inside fp16."""
    w = torch.randint(0, 256, rows_shape + (width // 256, 144), dtype=torch.uint8, device="cuda", generator=gen)
    w[..., 1] = (w[..., 1] & d_bits) | 0x0C
    w[..., 3] = (w[..., 3] & 0x03) | 0x0C
    return w.reshape(rows_shape + (width // 256 * 144,))


def extra_config3_small(strix, torch, cfg, steps, warmup):
    """Config 3 at the other token counts of its family (1 and 4): the same rotating layers, the first rows of their inputs."""
    out = {}
    n = len(cfg.layers)
    for t in (1, 4):
        def step(i):
            layer, wr, x = cfg.layers[i % n]
            layer.run_layer(x[:t], wr)
        sec = time_steps(torch, step, max(steps, 60), max(warmup, 12))
        u = statistics.mean(int(torch.unique(strix.route(x[:t], wr, cfg.K)[0]).numel()) for _, wr, x in cfg.layers)
        nbytes = u * 3 * cfg.I * Q4K_ROW(cfg.H) + cfg.E * cfg.H * 4 + t * (cfg.H * 2 + cfg.H * 4)
        out[f"config3_moe_decode_T{t}"] = {"us": sec * 1e6, "GBps": nbytes / sec / 1e9, "hbm_frac": nbytes / sec / 1e9 / HBM_PEAK_GBPS,
                                           "algorithmic_bytes": nbytes, "distinct_experts_mean": u}
    return out


def device_blocks(torch, gen, rows, blocks, block_bytes, scale_bytes, high):
    """Random quantized blocks [rows][blocks * block_bytes] whose fp16 scale fields (high bytes at `scale_bytes`) are small and finite."""
    w = torch.randint(0, 256, (rows, blocks, block_bytes), dtype=torch.uint8, device="cuda", generator=gen)
    for at in scale_bytes:
        w[..., at] = (w[..., at] & 0x03) | high
    return w.reshape(rows, -1)


def extra_config3_executor_formats(strix, torch, cfg, steps, warmup, with_cpu):
    """Config 3 (T rows) with the expert tensors in the other formats of the path: the reference host executor's own
    (gate/up Q4_K or Q5_K, down Q8_0 or Q5_1), which the compiled reference can run itself, and Q6_K down rows. GPU: the whole
    layer; CPU: the reference's Executor (its best ISA, every host thread) on the expert job of layer 0 (A8 rows in, rawdots
    out: no router, no combine)."""
    H, I, E, K, T = cfg.H, cfg.I, cfg.E, cfg.K, cfg.T
    gen = torch.Generator(device="cuda").manual_seed(5)
    out = {}
    combos = (("q4_k_gate_q8_0_down", strix.TYPE_Q4_K, strix.TYPE_Q8_0, 0), ("q5_k_gate_q5_1_down", strix.TYPE_Q5_K, strix.TYPE_Q5_1, 3),
              ("q4_k_gate_q6_k_down", strix.TYPE_Q4_K, strix.TYPE_Q6_K, None))
    for name, gate_type, down_type, ref_flags in combos:
        layers = []
        for layer, wr, x in cfg.layers:
            if gate_type == strix.TYPE_Q5_K:
                gate, up = (device_blocks(torch, gen, E * I, H // 256, 176, (1, 3), 0x10).reshape(E, I, -1) for _ in range(2))
            else:
                gate, up = layer.gate, layer.up
            if down_type == strix.TYPE_Q8_0:
                down = device_blocks(torch, gen, E * H, I // 32, 34, (1,), 0x14)
            elif down_type == strix.TYPE_Q5_1:
                down = device_blocks(torch, gen, E * H, I // 32, 24, (1, 3), 0x14)
            else:
                down = device_blocks(torch, gen, E * H, I // 256, 210, (209,), 0x08)
            layers.append((strix.MoeLayer(H, I, E, K, gate, up, down.reshape(E, H, -1), T, gate_type=gate_type, down_type=down_type), wr, x))
        n = len(layers)

        def step(i):
            layer, wr, x = layers[i % n]
            layer.run_layer(x, wr)
        sec = time_steps(torch, step, max(steps, 60), max(warmup, 12))
        entry = {"us": sec * 1e6}
        if int(sum(int(l.status.sum()) for l, _, _ in layers)):
            raise RuntimeError(f"{name}: a run set row status bits: the timing is void")
        if with_cpu and ref_flags is not None:
            import ctypes as C
            import orc
            R = orc.ref()
            if R is not None:
                layer, wr, x = layers[0]
                xn = x.cpu().numpy().astype(np.float32)
                ids, _, _, _ = orc.route(xn, wr.cpu().numpy(), K)
                c, d, s, _ = orc.quantize_a8(xn)
                gate, up, down = (t.cpu().numpy() for t in (layer.gate, layer.up, layer.down))
                asg = np.array([[t, k, ids[t, k]] for t in range(T) for k in range(K)], np.uint32)
                raw, status = np.zeros((T, K, H), np.float32), np.zeros(T, np.uint32)
                threads = orc.lib().orc_max_threads()
                R.ref_executor_run.restype = C.c_int
                pool = C.c_void_p(R.ref_executor_create(threads, 1))

                def run():
                    return R.ref_executor_run(pool, H, I, gate.ctypes.data_as(orc.u8p), up.ctypes.data_as(orc.u8p), down.ctypes.data_as(orc.u8p),
                                              ref_flags, c.ctypes.data_as(orc.i8p), d.ctypes.data_as(orc.f32p), s.ctypes.data_as(orc.i32p), T,
                                              asg.ctypes.data_as(orc.u32p), T * K, raw.ctypes.data_as(orc.f32p), C.c_uint64(K * H),
                                              status.ctypes.data_as(orc.u32p))
                if run() == 0:
                    times, t_end = [], time.perf_counter() + 4.0
                    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 200):
                        t0 = time.perf_counter()
                        run()
                        times.append(time.perf_counter() - t0)
                    layer.run_layer(x, wr)
                    torch.cuda.synchronize()
                    entry["cpu_reference"] = {"value": statistics.median(times) * 1e6, "unit": "us/expert job", "cores": threads, "kind": "reference",
                                              "isa": R.ref_executor_isa(pool).decode(),
                                              "sample": f"the reference's own Executor on layer 0's expert job, median of {len(times)} passes",
                                              "rawdots_equal_gpu_bits": bool(np.array_equal(raw.view(np.uint32), layer.rawdots[:T].cpu().numpy().view(np.uint32)))}
                R.ref_executor_destroy(pool)
        out[f"config3_moe_decode_T{T}_{name}"] = entry
        del layers
    return out


def extra_union_rows(strix, torch, steps, warmup):
    """The union rows form of the A8 entry points (R = 8 rows of a verify window; geometry and routes of the reference's device
    test, tests/hip_moe_a8_union_tests.hip:117-119: hidden = intermediate = 1536, 64 experts top-16, Q4_K gate / up, Q6_K down):
    probe + down quantise + down rows in three calls that read every distinct expert once, beside the same rows as eight
    single-row call triples. Weight sets rotate so that no pass finds its experts in the cache."""
    H, I, E, K, R = 1536, 1536, 64, 16, 8
    gen = torch.Generator(device="cuda").manual_seed(23)
    ids = torch.tensor([[(k * 5 + r * 3) % E for k in range(K)] for r in range(R)], dtype=torch.int32, device="cuda")
    x = torch.randn((R, H), device="cuda", generator=gen).to(torch.bfloat16)
    sets = []
    for _ in range(6):                                           # 6 x 0.36 GB of experts
        gate, up = device_q4k(torch, gen, (E, I), H), device_q4k(torch, gen, (E, I), H)
        down = device_blocks(torch, gen, E * H, I // 256, 210, (209,), 0x08).reshape(E, H, -1)
        un = strix.A8Decode(H, I, E, K, gate, up, down, rows=R, down_type=strix.TYPE_Q6_K)
        one = strix.A8Decode(H, I, E, K, gate, up, down, rows=1, down_type=strix.TYPE_Q6_K)
        un.input.copy_(x)
        un.routes.copy_(ids)
        sets.append((un, one))
    n = len(sets)

    def union_step(i):
        un = sets[i % n][0]
        un.enqueue_probe_union()
        un.enqueue_down_activation_quantize_union()
        un.enqueue_down_rawdots_union()

    def single_step(i):
        one = sets[i % n][1]
        for r in range(R):                                       # (the row's input and routes are in place: only the calls are timed)
            one.enqueue_probe()
            one.enqueue_down_activation_quantize()
            one.enqueue_down_rawdots()
    for _, one in sets:
        one.input.copy_(x[:1])
        one.routes.copy_(ids[:1])
    # the calls are shorter than their Python wrappers: one pass over the weight sets of each form is captured in a HIP graph
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graphs = []
    with torch.cuda.stream(side):
        for step in (union_step, single_step):
            for i in range(n):
                step(i)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for i in range(n):
                    step(i)
            graphs.append(graph)
    torch.cuda.synchronize()
    sec = time_steps(torch, lambda i: graphs[0].replay(), max(steps // 4, 10), 3) / n
    sec_single = time_steps(torch, lambda i: graphs[1].replay(), max(steps // 4, 10), 3) / n
    if any(int(un.status.item()) or int(one.status.item()) for un, one in sets):
        raise RuntimeError("union rows: a run set status bits: the timing is void")
    u = int(torch.unique(ids).numel())
    nbytes = u * (2 * I * Q4K_ROW(H) + H * (I // 256) * 210) + R * H * 2 + R * K * (3 * I * 4 + I * 1.25 + H * 4)
    return {"a8_union_rows_R8_q6_k_down": {"us": sec * 1e6, "us_as_8_single_row_calls": sec_single * 1e6, "distinct_experts": u, "assignments": R * K,
                                           "GBps": nbytes / sec / 1e9, "hbm_frac": nbytes / sec / 1e9 / HBM_PEAK_GBPS, "algorithmic_bytes": nbytes}}


def prefill_config4(strix, torch, gen, keep=False, reps=10):
    """BASELINE config 4: 4096 fp16 rows, hidden 4096, 256 routed Q4_K experts top-8 (router logits + N(0, 1.5) per-expert bias:
    Zipf-like load) of intermediate 2048, plus the always-on shared Q8_0 expert; router + shared expert + routed experts +
    ordered combine on the matrix cores (mi355_moe_enqueue_prefill_f16: exact integer operands, fp32 block scales and
    accumulation). FLOPs: the algorithmic 2 x rows x (8 + 1) x 3 x 2048 x 4096 + the router's."""
    H, I, E, K, T = 4096, 2048, 256, 8, 4096
    gate, up, down = (device_q4k(torch, gen, (E, I), H, 0x03), device_q4k(torch, gen, (E, I), H, 0x03), device_q4k(torch, gen, (E, H), I, 0x03))
    wr = torch.randn((E, H), device="cuda", generator=gen) * 0.02
    bias = torch.randn(E, device="cuda", generator=gen) * 1.5
    xp = torch.randn((T, H), device="cuda", generator=gen).to(torch.float16)
    layer = strix.MoeLayer(H, I, E, K, gate, up, down, T, prefill_f16=True)
    flops_experts, flops_router, flops_shared = 2.0 * T * K * 3 * I * H, 2.0 * T * E * H, 2.0 * T * 3 * I * H
    ids, wts, _ = strix.route(xp, wr, K, bias=bias)
    sec_route = time_steps(torch, lambda i: strix.route(xp, wr, K, bias=bias), 5, 2)
    sec_f16 = time_steps(torch, lambda i: layer.run_prefill_f16(xp, ids, wts), reps, 3)

    def q8(rows, width):
        w = torch.randint(0, 256, (rows, width // 32, 34), dtype=torch.uint8, device="cuda", generator=gen)
        w[..., 1] = (w[..., 1] & 0x03) | 0x14
        return w.reshape(rows, -1)
    sg, su, sd = q8(I, H), q8(I, H), q8(H, I)
    # the shared expert: a one-expert layer in the same prefill form, its output the base of the routed combine
    dense = strix.MoeLayer(H, I, 1, 1, sg.reshape(1, I, -1), su.reshape(1, I, -1), sd.reshape(1, H, -1), T, prefill_f16=True,
                           gate_type=strix.TYPE_Q8_0, down_type=strix.TYPE_Q8_0)
    zero_ids = torch.zeros((T, 1), dtype=torch.int32, device="cuda")
    ones = torch.ones((T, 1), dtype=torch.float32, device="cuda")
    sec_shared = time_steps(torch, lambda i: dense.run_prefill_f16(xp, zero_ids, ones), reps, 3)

    def whole(i):
        r_ids, r_wts, _ = strix.route(xp, wr, K, bias=bias)
        # the shared expert without its one-slot combine: its unweighted outputs are the routed combine's base
        shared = dense.run_prefill_f16(xp, zero_ids, ones, combine=strix.COMBINE_NONE).reshape(T, H)
        return layer.run_prefill_f16(xp, r_ids, r_wts, base=shared)
    sec_whole = time_steps(torch, whole, reps, 3)
    if int(layer.status.sum()) or int(dense.status.sum()):
        raise RuntimeError("config 4: the prefill run set row status bits (non-finite or out-of-range values): the timing is void")
    total = flops_experts + flops_router + flops_shared
    out = {
        "workload": "BASELINE config 4: 4096 fp16 rows, hidden 4096, 256 routed Q4_K experts top-8 (biased router) + 1 shared Q8_0 expert, intermediate 2048",
        "ms": sec_whole * 1e3, "TFLOPs": total / sec_whole / 1e12, "frac": total / sec_whole / MFMA_F16_PEAK_FLOPS, "peak": MFMA_F16_PEAK_FLOPS / 1e12,
        "unit": "TFLOP/s", "bound": "mfma", "dtype": "f16 operands, f32 accumulation", "algorithmic_flops": total,
        "kernel": "prefill_reg_kernel<0> (gate/up + SwiGLU) and <1> (down) of the routed Q4_K experts; prefill_f16_kernel for the shared Q8_0 expert",
        "experts_ms": sec_f16 * 1e3, "experts_TFLOPs": flops_experts / sec_f16 / 1e12, "experts_frac": flops_experts / sec_f16 / MFMA_F16_PEAK_FLOPS,
        "router_ms": sec_route * 1e3, "shared_expert_ms": sec_shared * 1e3, "shared_expert_TFLOPs": flops_shared / sec_shared / 1e12,
        "note": "FAST class (fp16 MFMA on exact integer operands sc*q, fp32 block scales and accumulation), tolerance 2e-3 against the exact-weight product; router exact-order"}
    # the routed experts of the same workload in the bit-exact integer-dot class (int8 matrix-core group dots, the reference's fp32
    # chain on the vector ALU), router included: what exactness costs beside the FAST class
    sec_int = time_steps(torch, lambda i: layer.run_layer(xp, wr, bias=bias), 3, 1)
    out["routed_experts_integer_class_ms"] = sec_int * 1e3
    if keep:
        # the same expert in the integer-dot class (A8 image, gate / up, SwiGLU + A8, down), for the comparison in --extra
        def shared(i):
            c, d, _, _ = strix.quantize_a8(xp)
            hc, hd, _, _, _ = strix.swiglu_quantize(strix.gemv_q8_0_a8(sg, c, d, H, I), strix.gemv_q8_0_a8(su, c, d, H, I))
            return strix.gemv_q8_0_a8(sd, hc, hd, I, H)
        out["shared_expert_integer_class_ms"] = time_steps(torch, shared, 3, 1) * 1e3
        return out, layer, xp, wr, bias
    return out


def extra_configs(strix, torch, steps, warmup):
    """BASELINE configs 1, 2, 4, 5 on synthetic full-entropy blocks; HBM-bound ones rotate over enough weight sets to stay cold."""
    gen = torch.Generator(device="cuda").manual_seed(11)
    out = {}
    # what the machine gives vendor kernels (not this library's code): a 1 GiB device copy and a large fp16 GEMM, as the
    # practical ceilings next to the published peaks the fractions below are quoted against
    src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(src)
    sec = time_steps(torch, lambda i: dst.copy_(src), 10, 3)
    out["probe_device_copy_1GiB"] = {"GBps_read_plus_write": 2.0 * src.numel() / sec / 1e9, "frac_of_hbm_peak": 2.0 * src.numel() / sec / 1e9 / HBM_PEAK_GBPS}
    del src, dst
    ga = torch.randn((8192, 8192), device="cuda", generator=gen).to(torch.float16)
    gb = torch.randn((8192, 8192), device="cuda", generator=gen).to(torch.float16)
    sec = time_steps(torch, lambda i: torch.matmul(ga, gb), 10, 3)
    out["probe_fp16_gemm_8192_vendor_library"] = {"TFLOPs": 2.0 * 8192 ** 3 / sec / 1e12, "frac_of_fp16_mfma_peak": 2.0 * 8192 ** 3 / sec / 2.5e15}
    del ga, gb
    # hand-written measurement kernels of the benchmark's own library (libmi355_bench_probes.so; not part of the product):
    probes = load_probes()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    # (a) the matrix cores on their own: a register-operand MFMA loop on every compute unit, with constant and with pseudo-random
    #     operands (the second is the ceiling a product on real data has under the chip's power limit)
    sink = torch.empty(512 * 1024, dtype=torch.float32, device="cuda")
    def mfma(rnd):
        flops = C.c_uint64(0)
        rc = probes.bench_probe_mfma_f16(20000, int(rnd), C.c_void_p(sink.data_ptr()), sink.numel(), C.byref(flops), stream)
        assert rc == 0, rc
        return flops.value
    for name, rnd in (("constant_operands", False), ("random_operands", True)):
        flops = mfma(rnd)
        sec = time_steps(torch, lambda i: mfma(rnd), 3, 1)
        out["probe_mfma_f16_register_loop_" + name] = {"TFLOPs": flops / sec / 1e12, "frac_of_fp16_mfma_peak": flops / sec / 2.5e15}
    del sink
    # (b) a read-only stream in the decode sweeps' own shape: one-wave workgroups, stages of 9,216 bytes, register loads or
    #     global -> LDS copies through a ring, contiguous or as 144-byte blocks of 64 rows; launches of the decode layer's sizes
    #     (1536 waves x 8 stages = the gate / up launch, 2048 x 3 = the down launch) and a 1 GiB stream. Every step reads a
    #     different part of a 4 GiB buffer, so nothing is cache resident.
    pool = torch.randint(0, 256, (4 << 30,), dtype=torch.uint8, device="cuda", generator=gen)
    words = torch.empty(1 << 16, dtype=torch.int32, device="cuda")
    reads = {}
    for label, waves, stages in (("gate_up_launch_1536x8", 1536, 8), ("down_launch_2048x3", 2048, 3), ("stream_1GiB_14563x8", 14563, 8), ("stream_1GiB_1536x76", 1536, 76)):
        nbytes = waves * stages * 9216
        slots = pool.numel() // nbytes
        for mode, mname in ((0, "registers"), (1, "lds_ring_contiguous"), (2, "lds_ring_144B_of_64_rows")):
            for depth in (2, 4):
                def run(i):
                    at = (i % slots) * nbytes
                    rc = probes.bench_probe_read_stream(C.c_void_p(pool.data_ptr() + at), waves, stages, mode, depth, C.c_void_p(words.data_ptr()), stream)
                    assert rc == 0, rc
                sec = time_steps(torch, run, 12 if nbytes < (1 << 29) else 4, 3)
                reads[f"{label}_{mname}_depth{depth}"] = {"us": sec * 1e6, "GBps": nbytes / sec / 1e9, "frac_of_hbm_peak": nbytes / sec / 1e9 / HBM_PEAK_GBPS}
    out["probe_read_only_stream"] = reads
    del pool, words
    # config 1: Q8_0 4096 x 4096 GEMV, one fp32 row
    n = 4096
    sets = []
    for _ in range(24):      # 24 x 17.8 MB = 428 MB
        w = torch.randint(0, 256, (n, n // 32, 34), dtype=torch.uint8, device="cuda", generator=gen)
        w[..., 1] = (w[..., 1] & 0x03) | 0x14
        sets.append(w.reshape(n, -1))
    x = torch.randn((1, n), device="cuda", generator=gen)
    c, d, _, _ = strix.quantize_a8(x)
    y = torch.zeros((1, n), device="cuda")
    # one launch is shorter than a Python call: the 24 launches (one per weight set) are captured in a HIP graph and replayed
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        for w in sets:
            strix.gemv_q8_0_a8(w, c, d, n, n, out=y)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for w in sets:
                strix.gemv_q8_0_a8(w, c, d, n, n, out=y)
    torch.cuda.synchronize()
    sec = time_steps(torch, lambda i: graph.replay(), max(steps // 4, 10), 3) / len(sets)
    nbytes = n * (n // 32) * 34 + n * 1.125 + n * 4
    out["config1_q8_0_gemv_4096x4096"] = {"us": sec * 1e6, "GBps": nbytes / sec / 1e9, "hbm_frac": nbytes / sec / 1e9 / HBM_PEAK_GBPS,
                                          "algorithmic_bytes": nbytes}
    del sets
    # config 2: dense Q4_K FFN 27648 x 5120, B = 1, 4, 8 (3 rotating weight sets = 717 MB)
    H, I = 5120, 27648
    layers = [strix.MoeLayer(H, I, 1, 1, device_q4k(torch, gen, (1, I), H), device_q4k(torch, gen, (1, I), H), device_q4k(torch, gen, (1, H), I), 8, intermediates=True)
              for _ in range(3)]
    for B in (1, 4, 8):
        xb = torch.randn((B, H), device="cuda", generator=gen).to(torch.float16)
        ids = torch.zeros((B, 1), dtype=torch.int32, device="cuda")
        w1 = torch.ones((B, 1), dtype=torch.float32, device="cuda")
        sec = time_steps(torch, lambda i: layers[i % 3].run(xb, ids, w1), max(steps // 4, 10), max(warmup // 4, 3))
        nbytes = 3 * I * (H // 256) * 144 + B * (H * 2 + H * 4)
        out[f"config2_dense_q4k_ffn_B{B}"] = {"us": sec * 1e6, "GBps": nbytes / sec / 1e9, "hbm_frac": nbytes / sec / 1e9 / HBM_PEAK_GBPS,
                                              "algorithmic_bytes": nbytes}
    del layers
    # RMSNorm in front of the block (the third entry of the reference's CPU kernel table): 4096 rows of 4096 fp32
    xn = torch.randn((4096, 4096), device="cuda", generator=gen)
    wn = torch.randn(4096, device="cuda", generator=gen)
    sec = time_steps(torch, lambda i: strix.rmsnorm_f32(xn, wn), max(steps // 4, 10), max(warmup // 4, 3))
    nbytes = 2 * xn.numel() * 4 + wn.numel() * 4
    out["rmsnorm_f32_4096x4096"] = {"us": sec * 1e6, "GBps": nbytes / sec / 1e9, "hbm_frac": nbytes / sec / 1e9 / HBM_PEAK_GBPS, "algorithmic_bytes": nbytes}
    del xn, wn
    # config 5: expert-TP rank 0 of 2, 16 rows, hidden 6144, 160 experts top-8, intermediate 2560 / 2
    H, I, E, K, T = 6144, 2560, 160, 8, 16
    grb, drb = H // 256 * 144, I // 256 * 144
    layer = strix.MoeLayer(H, I // 2, E, K, device_q4k(torch, gen, (E, I), H), device_q4k(torch, gen, (E, I), H), device_q4k(torch, gen, (E, H), I), T,
                           gate_expert_stride=I * grb, gate_row_stride=grb, down_expert_stride=H * drb, down_row_stride=drb)
    wr = torch.randn((E, H), device="cuda", generator=gen) * 0.02
    xs = [torch.randn((T, H), device="cuda", generator=gen).to(torch.float16) for _ in range(4)]
    sec = time_steps(torch, lambda i: layer.run_layer(xs[i % 4], wr, combine=strix.COMBINE_MULADD_ASC), max(steps // 4, 10), max(warmup // 4, 3))
    u = statistics.mean(int(torch.unique(strix.route(xv, wr, K)[0]).numel()) for xv in xs)
    nbytes = u * 3 * (I // 2) * grb + E * H * 4 + T * H * 6
    out["config5_tp_rank_shard_T16"] = {"us": sec * 1e6, "GBps": nbytes / sec / 1e9, "hbm_frac": nbytes / sec / 1e9 / HBM_PEAK_GBPS,
                                        "algorithmic_bytes": nbytes, "distinct_experts_mean": u}
    del layer
    # config 4 (the 4096-row prefill) on the matrix cores, and the same work in the bit-exact integer-dot class
    pf, layer, xp, wr, bias = prefill_config4(strix, torch, gen, keep=True)
    out["config4_prefill_T4096_f16_mfma"] = pf
    H, I, E, K, T = 4096, 2048, 256, 8, 4096
    flops_experts, flops_router = 2.0 * T * K * 3 * I * H, 2.0 * T * E * H
    sec = time_steps(torch, lambda i: layer.run_layer(xp, wr, bias=bias), 2, 1)
    out["config4_prefill_T4096_integer_class"] = {
        "ms": sec * 1e3, "TFLOPs": (flops_experts + flops_router) / sec / 1e12, "algorithmic_flops": flops_experts + flops_router,
        "note": "same work in the bit-exact integer-dot class: int8 matrix-core group dots, the fp32 chain on the vector ALU (router included)"}
    return out


def load_probes():
    """The benchmark's own measurement kernels (strix-halo-engine-lab_amd/bench_probes/probes.hip), built by __graft_entry__.build()."""
    lib = C.CDLL(os.path.join(ROOT, "strix-halo-engine-lab_amd", "libmi355_bench_probes.so"))
    lib.bench_probe_read_stream.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]
    lib.bench_probe_mfma_f16.argtypes = [C.c_uint32, C.c_uint32, C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]
    return lib


def time_steps(torch, fn, steps, warmup):
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        fn(warmup + i)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def host_cpu_info(threads):
    """Host CPU model, the vector ISA flags that matter to the reference's CPU kernels, and a plain multi-thread read-bandwidth
    ceiling (method of the reference's scripts/bench/residency/cpu_expert_bench.cpp:131-147)."""
    import ctypes as C
    import orc
    model, flags = "unknown", set()
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name") and model == "unknown":
                model = line.split(":", 1)[1].strip()
            if line.startswith("flags") and not flags:
                flags = set(line.split(":", 1)[1].split())
    except OSError:
        pass
    isa = [f for f in ("avx2", "avx_vnni", "avx512f", "avx512bw", "avx512_vnni", "amx_int8") if f in flags]
    buf = np.ones(1 << 27, np.uint64)      # 1 GiB
    L = orc.lib()
    L.orc_read_seconds.restype = C.c_double
    L.orc_read_seconds.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p]
    L.orc_read_seconds(buf.ctypes.data, buf.size, 1, threads, None)
    sec = L.orc_read_seconds(buf.ctypes.data, buf.size, 4, threads, None) / 4.0
    return {"cpu_model": model, "isa_flags": isa, "read_bandwidth_GBps": buf.nbytes / sec / 1e9, "read_bandwidth_threads": threads}


def reference_executor_config3(cfg, torch, strix, budget_s=4.0):
    """The compiled reference's own Executor (its best ISA, every host thread) on layer 0's expert job of the same geometry with
    the down tensors in Q8_0 - the executor has no Q4_K down rows (src/cpu/core/routed_expert.hpp:28), so the gate/up tensors,
    tokens and routes are the workload's and only the down tensor's format differs. None where oracle/_ref was not built."""
    import ctypes as C
    import orc
    R = orc.ref()
    if R is None:
        return None
    layer, wr, x = cfg.layers[0]
    H, I, E, K, T = cfg.H, cfg.I, cfg.E, cfg.K, cfg.T
    gen = torch.Generator(device="cuda").manual_seed(5)
    down = device_blocks(torch, gen, E * H, I // 32, 34, (1,), 0x14).cpu().numpy()
    gate, up = layer.gate.cpu().numpy(), layer.up.cpu().numpy()
    xn = x.cpu().numpy().astype(np.float32)
    ids, _, _, _ = orc.route(xn, wr.cpu().numpy(), K)
    c, d, s, _ = orc.quantize_a8(xn)
    asg = np.array([[t, k, ids[t, k]] for t in range(T) for k in range(K)], np.uint32)
    raw, status = np.zeros((T, K, H), np.float32), np.zeros(T, np.uint32)
    threads = orc.lib().orc_max_threads()
    R.ref_executor_run.restype = C.c_int
    pool = C.c_void_p(R.ref_executor_create(threads, 1))

    def run():
        return R.ref_executor_run(pool, H, I, gate.ctypes.data_as(orc.u8p), up.ctypes.data_as(orc.u8p), down.ctypes.data_as(orc.u8p), 0,
                                  c.ctypes.data_as(orc.i8p), d.ctypes.data_as(orc.f32p), s.ctypes.data_as(orc.i32p), T,
                                  asg.ctypes.data_as(orc.u32p), T * K, raw.ctypes.data_as(orc.f32p), C.c_uint64(K * H),
                                  status.ctypes.data_as(orc.u32p))
    out = None
    if run() == 0:
        times, t_end = [], time.perf_counter() + budget_s
        while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 200):
            t0 = time.perf_counter()
            run()
            times.append(time.perf_counter() - t0)
        out = {"value": statistics.median(times) * 1e6, "unit": "us/expert job", "cores": threads, "kind": "reference",
               "isa": R.ref_executor_isa(pool).decode(),
               "sample": f"the reference's Executor on layer 0's expert job (gate/up/SwiGLU/down of {T * K} assignments; no router, no combine) "
                         f"with the workload's Q4_K gate/up tensors and a Q8_0 down tensor, median of {len(times)} passes"}
    R.ref_executor_destroy(pool)
    return out


def cpu_baseline_config3(cfg, budget_s=12.0):
    """The CPU oracle (port of the reference's CPU path) on layer 0 of the same workload, all host threads."""
    import orc
    layer, wr, x = cfg.layers[0]
    H, I, E, K, T = cfg.H, cfg.I, cfg.E, cfg.K, cfg.T
    gate, up, down = (t.cpu().numpy() for t in (layer.gate, layer.up, layer.down))
    xn, wrn = x.cpu().numpy().astype(np.float32), wr.cpu().numpy()
    threads = orc.lib().orc_max_threads()

    def run():
        ids, wts, _, _ = orc.route(xn, wrn, K, threads=threads)
        c, d, s, _ = orc.quantize_a8(xn)
        r = orc.routed_experts(H, I, K, gate, up, down, orc.Q4_K, c, d, s, ids, threads=threads, want_intermediates=False)
        return orc.combine(orc.COMBINE_FMA_SLOT, wts, ids, r.rawdots)

    run()
    times, t_end = [], time.perf_counter() + budget_s
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 50):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    med = statistics.median(times)
    return {"value": med * 1e6, "unit": "us/layer", "cores": threads, "kind": "port",
            "sample": f"layer 0 of the same config-3 workload (T={T}), median of {len(times)} passes after one warm-up; "
                      "C restatement of the reference CPU path (Q4_K rows: byte dot-product instruction and the sub-block chain in vector lanes where the host has AVX-VNNI, same bits as the plain loop), "
                      "OpenMP over (assignment, 32-output group) and (assignment, output)"}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU's share: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import torch
    from __graft_entry__ import load_package
    strix = load_package()
    strix.require_gpu()
    torch.cuda.set_device(0)

    # every rotating layer is run in the warm-up: a layer's first call pays for things that are not decode throughput (first touch
    # of its workspace, page-table walks over its 340 MB of weights: 30 - 80 us once, 1.5 - 4 us per step over 20 steps)
    n_layers = max(2, min(args.layers, args.warmup)) if args.warmup > 0 else args.layers
    cfg = Config3(strix, torch, n_layers, args.tokens)
    u_list = cfg.distinct_experts()
    u_mean = sum(u_list) / len(u_list)

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()

    sec = time_steps(torch, cfg.step, args.steps, args.warmup)

    # the staged entry points one by one, an event pair around each call: launch latency and the gap to the next call are
    # inside these figures (the kernels' own durations are in profiles/ and, for the projection, in roofline.avg_launch_us)
    events = []
    for i in range(args.warmup):
        cfg.staged_step(i, [])
    torch.cuda.synchronize()
    for i in range(args.steps):
        cfg.staged_step(args.warmup + i, events)
    torch.cuda.synchronize()
    names = ("route", "prologue", "csr", "project", "down", "merge")
    staged_call_us = {n: statistics.mean(m[k].elapsed_time(m[k + 1]) for m in events) * 1e3 for k, n in enumerate(names)}
    project_us = cfg.project_launch_us(max(args.steps // len(cfg.layers), 4))
    front_us, back_us = cfg.halves_launch_us(max(args.steps // len(cfg.layers), 4))
    achieved = cfg.front_bytes(u_mean) / (front_us * 1e-6) / 1e9
    layer_gbps = cfg.layer_bytes(u_mean) / sec / 1e9

    out = {
        "metric": "moe_decode_us_per_layer", "value": sec * 1e6, "unit": "us/layer", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": sec * 1e3, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "i8", "data": "synthetic",
        "config": {"workload": f"BASELINE config 3: MoE decode layer, Q4_K experts, hidden 2048, 128 experts, softmax router top-8, "
                               f"intermediate 768, {args.tokens} fp16 tokens, router + experts + combine, {n_layers} rotating layers (cold cache)",
                   "tokens": args.tokens, "distinct_experts_mean": u_mean},
        "hbm_GBps_layer": layer_gbps, "hbm_frac_layer": layer_gbps / HBM_PEAK_GBPS,
        "layer_algorithmic_bytes": cfg.layer_bytes(u_mean), "staged_call_us": staged_call_us,
        "launch_us": {"front (layer_front_kernel)": front_us, "back (down rows + combine: down_merge_flat_kernel)": back_us,
                      "staged gate/up alone (project_wave_kernel)": project_us},
        "roofline": {"bound": "hbm", "kernel": "layer_front_kernel (early routes + A8 prologue + exact router + gate/up + SwiGLU + A8 re-quantise)",
                     "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
                     "traffic": FRONT_TRAFFIC_BYTES_DEFAULT if args.tokens == 8 else None,
                     "traffic_source": FRONT_TRAFFIC_SOURCE,
                     "algorithmic_bytes_per_launch": cfg.front_bytes(u_mean), "avg_launch_us": front_us,
                     "timing": "HIP events on the launch stream around the front launches (mi355_moe_enqueue_layer_front) of all rotating layers enqueued back to back"},
    }
    if args.extra:
        small = extra_config3_small(strix, torch, cfg, args.steps, args.warmup) if args.tokens >= 4 else {}
        small.update(extra_config3_executor_formats(strix, torch, cfg, args.steps, args.warmup, not args.no_cpu))
        del cfg.layers[1:]
        small.update(extra_union_rows(strix, torch, args.steps, args.warmup))
        out["extra"] = {**small, **extra_configs(strix, torch, args.steps, args.warmup)}
    if args.extra:
        out["prefill"] = out["extra"]["config4_prefill_T4096_f16_mfma"]
    elif not args.no_prefill:
        # the second target of the metric: the 4096-row prefill on the matrix cores (BASELINE config 4, whole layer)
        del cfg.layers[1:]
        torch.cuda.empty_cache()
        out["prefill"] = prefill_config4(strix, torch, torch.Generator(device="cuda").manual_seed(11))
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_config3(cfg)
        out["cpu_baseline"]["reference_executor"] = reference_executor_config3(cfg, torch, strix)
        out["cpu_baseline"]["host"] = host_cpu_info(out["cpu_baseline"]["cores"])
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
