// Routed experts (and a dense FFN as the one-expert case) on the matrix-core sweep of q4k_mma.hpp, for work items of 3..32
// activation rows: one workgroup per (work item, 32 outputs).
//   project: the gate tile and the up tile of the same 32 features share the activation rows of a sweep; the epilogue is
//            the reference's SwiGLU + A8 re-quantisation of the 32-value group (src/cpu/core/routed_expert.cpp:147-170, :403-427).
//   down:    32 hidden outputs against the A8 image of h (src/cpu/core/routed_expert.cpp:429-447, src/moe_a8_down_contract.cpp:146).
// An item longer than 2 NAL rows is served in chunks; the second and later sweeps of the tile's weights come from the cache.
// dense_rows > 0: no plan, expert 0, assignment i = row i; blockIdx.y picks a chunk of 2 NAL rows.
// (Included inside namespace strix950, after the plan helpers and RowsK accessors it uses.)
#pragma once

struct MmaItem { uint32_t e, begin, end; };
__device__ __forceinline__ MmaItem mma_item(const mi355_moe_weights& w, const RowsK& r, uint32_t assignments, uint32_t dense_rows, uint32_t width) {
    if (dense_rows) {                                       // one chunk of the batch per blockIdx.y
        const uint32_t begin = blockIdx.y * width, end = begin + width;
        return {0U, begin, end < dense_rows ? end : dense_rows};
    }
    const WorkItem item = work_item(w, r, plan_items_at(w.experts, assignments), blockIdx.y);
    return {static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(item.e)), static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(item.begin)),
            static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(item.end))};
}

template <int NAL, int DEPTH>
__global__ __launch_bounds__(256) void q4k_mma_project_kernel(mi355_moe_weights w, RowsK r, uint32_t assignments, uint32_t dense_rows) {
    constexpr uint32_t ACTS = mma_acts<NAL>();
    static_assert(mma_ring_bytes<NAL, 2, DEPTH, 1>() >= 4U * 2U * NAL * 256U, "the ring doubles as the reduction buffer");
    __shared__ __attribute__((aligned(16))) uint8_t ring_mem[mma_ring_bytes<NAL, 2, DEPTH, 1>()];
    const MmaItem item = mma_item(w, r, assignments, dense_rows, ACTS);
    if (item.begin == item.end) return;
    const uint32_t order_at = plan_order_at(w.experts), grp = blockIdx.x, lane = threadIdx.x & 63U, j = lane & 31U, h = lane >> 5;
    const size_t base = static_cast<size_t>(item.e) * w.gate_expert_stride + static_cast<size_t>(grp * 32U) * w.gate_row_stride;
    const uint8_t* const wrows[2] = {w.gate + base, w.up + base};
    const bool planned = !dense_rows;
    for (uint32_t c0 = item.begin; c0 < item.end; c0 += ACTS) {
        const uint32_t n = item.end - c0 < ACTS ? item.end - c0 : ACTS;
        const auto slot_of = [&](uint32_t a) { return planned ? ordered(r, order_at, c0 + a) : c0 + a; };       // assignment index
        const auto acts = [&](uint32_t a) {
            const uint32_t row = r.row_of(slot_of(a));
            return MmaActRow{reinterpret_cast<const uint8_t*>(r.in.codes_of(row)), reinterpret_cast<const uint8_t*>(r.in.deltas_of(row)),
                             reinterpret_cast<const uint8_t*>(r.in.sums_of(row))};
        };
        float acc[2][NAL];
        mma_sweep<NAL, DEPTH, 1, 2>((lds_u8*)ring_mem, nullptr, wrows, w.gate_row_stride, w.hidden / 256U, acts, n, acc);
        mma_reduce<NAL, 2>((lds_f32*)ring_mem, acc, n, [&](uint32_t v, const float (&value)[2]) {
            // lane (feature j, half h) holds gate and up of activation row 2v + h; a half past the chunk computes on and stores nothing
            const uint32_t a = 2U * v + h;
            const bool live = a < n;
            const uint32_t sidx = slot_of(live ? a : 0U);
            const float g = value[0], u = value[1];
            float gc = g, uc = u;
            swiglu_clamp(gc, uc, w.swiglu_limit);
            const float hv = (gc / (1.0F + exp_of(w.exp_kind, -gc))) * uc;
            const uint32_t at_out = grp * 32U + j;
            if (live) {
                if (r.gate_out) r.inter_of(r.gate_out, sidx)[at_out] = g;
                if (r.up_out) r.inter_of(r.up_out, sidx)[at_out] = u;
                if (r.h_out) r.inter_of(r.h_out, sidx)[at_out] = hv;
            }
            if (!r.h.codes) return;             // projection only (the probe form): no A8 image of h
            const int bad = or32_i((finite_f(g) && finite_f(u) && finite_f(hv)) ? 0 : 1);
            const float amax = max32(__builtin_fabsf(hv));
            const bool tiny = amax > 0.0F && amax < 0x1p-119F;
            const float dl = (amax == 0.0F || tiny) ? 1.0F : amax / 127.0F;
            const int code = a8_code(hv, dl, tiny);
            const int sum = sum32_i(code);
            if (!live) return;
            if (bad) {
                if (j == 0) {
                    atomicOr(r.status_of(r.row_of(sidx)), r.nonfinite_bit);
                    atomicOr(r.job_status, static_cast<uint32_t>(MI355_STATUS_NONFINITE_PROJECTION));
                }
                return;
            }
            r.h_codes_of(sidx)[at_out] = static_cast<int8_t>(code);
            if (j == 0) {
                r.h_deltas_of(sidx)[grp] = dl;
                r.h_sums_of(sidx)[grp] = sum;
            }
        });
    }
}

// GATE_UP: the same sweep over gate (blockIdx.z = 0) or up (1) rows against the input image, raw values out to the gate / up
// intermediates - the dense FFN's projection when that workspace exists (two launches' worth of narrow workgroups fill the
// compute units better than the fused form's wide ones: 27648 x 5120, 8 rows: 54 + 5 us against 70 us).
template <int NAL, int DEPTH, int TEAMS, bool GATE_UP = false>
__global__ __launch_bounds__(256 * TEAMS) void q4k_mma_down_kernel(mi355_moe_weights w, RowsK r, uint32_t assignments, uint32_t dense_rows) {
    constexpr uint32_t ACTS = mma_acts<NAL>();
    static_assert(mma_ring_bytes<NAL, 1, DEPTH, TEAMS>() >= 4U * NAL * 256U, "the ring doubles as the reduction buffer");
    __shared__ __attribute__((aligned(16))) uint8_t ring_mem[mma_ring_bytes<NAL, 1, DEPTH, TEAMS>()];
    __shared__ float xbuf_mem[mma_exchange_floats<NAL, TEAMS>()];
    const MmaItem item = mma_item(w, r, assignments, dense_rows, ACTS);
    if (item.begin == item.end) return;
    if (!GATE_UP && (*r.job_status & MI355_STATUS_NONFINITE_PROJECTION)) return;
    const uint32_t order_at = plan_order_at(w.experts), row0 = blockIdx.x * kMmaRows, lane = threadIdx.x & 63U;
    const uint8_t* const wrows[1] = {
        GATE_UP ? (blockIdx.z ? w.up : w.gate) + static_cast<size_t>(item.e) * w.gate_expert_stride + static_cast<size_t>(row0) * w.gate_row_stride
                : w.down + static_cast<size_t>(item.e) * w.down_expert_stride + static_cast<size_t>(row0) * w.down_row_stride};
    const A8Image& img = GATE_UP ? r.in : r.h;
    float* const inter = blockIdx.z ? r.up_out : r.gate_out;
    const bool planned = !dense_rows;
    for (uint32_t c0 = item.begin; c0 < item.end; c0 += ACTS) {
        const uint32_t n = item.end - c0 < ACTS ? item.end - c0 : ACTS;
        const auto slot_of = [&](uint32_t a) { return planned ? ordered(r, order_at, c0 + a) : c0 + a; };
        const auto acts = [&](uint32_t a) {
            const uint32_t i = GATE_UP ? r.row_of(slot_of(a)) : slot_of(a);
            return MmaActRow{reinterpret_cast<const uint8_t*>(img.codes_of(i)), reinterpret_cast<const uint8_t*>(img.deltas_of(i)),
                             reinterpret_cast<const uint8_t*>(img.sums_of(i))};
        };
        float acc[1][NAL];
        mma_sweep<NAL, DEPTH, TEAMS, 1>((lds_u8*)ring_mem, (lds_f32*)xbuf_mem, wrows, GATE_UP ? w.gate_row_stride : w.down_row_stride,
                                        (GATE_UP ? w.hidden : w.ffn) / 256U, acts, n, acc);
        mma_reduce<NAL, 1>((lds_f32*)ring_mem, acc, n, [&](uint32_t v, const float (&value)[1]) {
            const uint32_t a = 2U * v + (lane >> 5);
            if (a >= n) return;
            if (GATE_UP) r.inter_of(inter, slot_of(a))[row0 + (lane & 31U)] = value[0];
            else {
                r.rawdots_of(slot_of(a), w.hidden)[row0 + (lane & 31U)] = value[0];
                if (r.top1_form) r.publish_top1(slot_of(a), row0 + (lane & 31U), value[0]);      // (top-1: assignment = row)
            }
        });
    }
}
