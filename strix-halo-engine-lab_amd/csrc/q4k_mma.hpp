// Q4_K x A8 rows for a dense matrix against 3..16 activation rows: the exact group dots come from the int8 matrix cores,
// the reference's fp32 chain stays on the vector ALU.
//
// A workgroup (4 wavefronts) owns 32 weight rows. Wavefront p owns the reference's pair accumulator p of those rows
// (sub-blocks 2p and 2p + 1 of every super-block) - the four pair chains of a row are independent, K is never split.
// Per super-block a wavefront issues two v_mfma_i32_32x32x32_i8: operand B = 32 weight rows x the 32 nibbles of one
// sub-block (lane (row j, half h) carries elements 16h .. 16h + 15, expanded to bytes), operand A = 32 activation slots x the
// same 32 codes (lane (slot i, half h) carries codes 16h .. 16h + 15 of its row). Both operands put element k in the same
// register byte, so whatever order the core walks K in, a product pairs weight k with code k; an integer sum has no order.
// The 32 x 32 result leaves lane (j, h) with its row's dots against the slots 8 (v / 4) + 4h + v % 4, v = 0..15; activation
// row a sits in slot v = a / 2 of half h = a % 2, so the lane reads rows h, 2 + h, 4 + h, ... from result registers 0, 1, 2, ...
// and every lane of the wavefront does chain work for NAL = ceil(rows / 2) activation rows.
//
// Chain per (row, activation row, sub-block) - src/cpu/core/routed_expert.cpp:73-108 == src/moe_q4k_a8_contract.cpp:126-140:
//   u = (d * scale) * float(dot); v = (dmin * min) * float(code sum); x = delta * (u - v); acc[p] += x[2p] + x[2p + 1];
//   value = (acc[0] + acc[1]) + (acc[2] + acc[3]).
// delta and code sum depend on (activation row, sub-block) only: every quad of lanes keeps the four values of the wavefront's
// two sub-blocks (delta 2p, delta 2p + 1, sum 2p, sum 2p + 1) in its four lanes and the multiplies take them by quad
// broadcast (a DPP operand, no instruction of its own).
//
// Data path: a stage is one super-block of the 32 rows (4,608 bytes, rows back to back: a row is 144 = 128 + 16 bytes, so eight
// neighbouring rows read eight different 16-byte bank groups), the 256 codes of every activation row (piece t of row a at
// position (t + a) % 16 of its 16 pieces, which spreads eight rows over the bank groups) and one table piece per row
// (8 deltas, 8 sums). Everything arrives by global_load_lds_dwordx4 into a ring of DEPTH slots shared by the workgroup: a
// wavefront waits for its own copies (counted s_waitcnt vmcnt), the workgroup barrier publishes all of them, and the slot
// consumed before the barrier is refilled after it.
#pragma once
#include "q4k_pairs.hpp"

namespace strix950 {

typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
typedef int32_t i32x16 __attribute__((ext_vector_type(16)));

constexpr uint32_t kMmaRows = 32;
template <int NAL> constexpr uint32_t mma_acts() { return 2U * NAL; }                         // activation slots served (multiple of 4)
template <int NAL> constexpr uint32_t mma_code_copies() { return mma_acts<NAL>() / 4U; }      // 1 KiB = 4 rows x 256 codes
template <int NAL> constexpr uint32_t mma_copies() { return 5U + mma_code_copies<NAL>() + 1U; }   // weights 4.5 (5), codes, table
template <int NAL> constexpr uint32_t mma_slot_bytes() { return 1024U * mma_copies<NAL>(); }

// Workgroup barrier that orders LDS traffic only (__syncthreads() would also wait for every copy in flight, i.e. drain the
// ring at each stage): this wavefront's LDS reads and writes complete, then the barrier; arrivals of copies are awaited by count.
__device__ __forceinline__ void mma_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// One global -> LDS copy of 16 bytes per lane (lane l lands at lds_at + 16 l), issued as plain instructions: told about the copy,
// the compiler would hold every later LDS read until all copies in flight have landed. Arrival is awaited by count instead.
__device__ __forceinline__ void mma_copy16(const uint8_t* src, lds_u8* lds_at) {
    const uint32_t at = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds_at)));
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(at), "v"(src) : "memory", "m0");
}
template <int N> __device__ __forceinline__ void mma_wait() { asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory"); }
template <int N> __device__ __forceinline__ void mma_wait_n(uint32_t ahead) {   // at most N * ahead copies still in flight
    switch (ahead) {
    case 0: mma_wait<0>(); break;
    case 1: mma_wait<N>(); break;
    case 2: mma_wait<2 * N>(); break;
    case 3: mma_wait<3 * N>(); break;
    case 4: mma_wait<4 * N>(); break;
    case 5: mma_wait<5 * N>(); break;
    case 6: mma_wait<6 * N>(); break;
    default: mma_wait<7 * N>(); break;
    }
}

// Activation row served by operand-A slot i (the inverse of "row a -> result register a / 2 of half a % 2"); slots past the
// served rows repeat earlier rows (their results are never read).
template <int NAL> __device__ __forceinline__ uint32_t mma_slot_act(uint32_t i) {
    const uint32_t v = 4U * (i >> 3) + (i & 3U), h = (i >> 2) & 1U;
    return (2U * v + h) % mma_acts<NAL>();
}

// Per-lane byte offsets into a ring slot (constant over the sweep).
struct MmaLane {
    uint32_t head, quants, even, odd, table;
    bool sum_lane;
};

// The LDS operands of one landed super-block, in registers.
template <int NAL>
struct MmaOperands {
    u32x4 hd, q, a_even, a_odd;
    int32_t tab[NAL];
    __device__ __forceinline__ void load(const lds_u8* slot, const MmaLane& o) {
        typedef const __attribute__((address_space(3))) u32x4 lds_u32x4;
        typedef const __attribute__((address_space(3))) int32_t lds_i32;
        hd = *(lds_u32x4*)(slot + o.head);
        q = *(lds_u32x4*)(slot + o.quants);
        a_even = *(lds_u32x4*)(slot + o.even);
        a_odd = *(lds_u32x4*)(slot + o.odd);
#pragma unroll
        for (int v = 0; v < NAL; ++v) tab[v] = *(lds_i32*)(slot + o.table + 128U * v);
    }
};

// One super-block: the wavefront's two group dots of its 32 rows against every activation slot, then the lane's NAL chain
// terms x[2P] + x[2P + 1]. P is the wavefront's pair, a template argument so that the scale / min unpacking has constant
// shifts.
template <int NAL, int P>
__device__ __forceinline__ void mma_stage_terms(const lds_u8* slot, const MmaLane& o, float (&term)[NAL]) {
    MmaOperands<NAL> r;
    r.load(slot, o);
    const u32x4 lo = r.q & 0x0f0f0f0fU, hi = (r.q >> 4) & 0x0f0f0f0fU;
    const i32x16 zero = {0};
    const i32x16 dot_even = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, r.a_even), __builtin_bit_cast(i32x4, lo), zero, 0, 0, 0);
    const i32x16 dot_odd = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, r.a_odd), __builtin_bit_cast(i32x4, hi), zero, 0, 0, 0);
    uint32_t s0, m0, s1, m1;
    q4k_factors<2 * P>(r.hd, s0, m0);
    q4k_factors<2 * P + 1>(r.hd, s1, m1);
    const float d = half_bits_to_float(r.hd.x & 0xffffU), dm = half_bits_to_float(r.hd.x >> 16);
    const float D0 = d * static_cast<float>(s0), M0 = dm * static_cast<float>(m0);
    const float D1 = d * static_cast<float>(s1), M1 = dm * static_cast<float>(m1);
    int32_t tab[NAL];
#pragma unroll
    for (int v = 0; v < NAL; ++v) tab[v] = r.tab[v];
    if (o.sum_lane) {                                       // quad lanes 2, 3 hold code sums: to float, once
#pragma unroll
        for (int v = 0; v < NAL; ++v) tab[v] = __builtin_bit_cast(int32_t, static_cast<float>(tab[v]));
    }
#pragma unroll
    for (int v = 0; v < NAL; ++v) {
        const float e0 = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(tab[v], 0x00, 0xF, 0xF, true));
        const float e1 = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(tab[v], 0x55, 0xF, 0xF, true));
        const float f0 = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(tab[v], 0xAA, 0xF, 0xF, true));
        const float f1 = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(tab[v], 0xFF, 0xF, 0xF, true));
        const float u0 = D0 * static_cast<float>(dot_even[v]), v0 = M0 * f0;
        const float u1 = D1 * static_cast<float>(dot_odd[v]), v1 = M1 * f1;
        const float x0 = e0 * (u0 - v0), x1 = e1 * (u1 - v1);
        term[v] = x0 + x1;
    }
}

// TEAMS > 1 (a matrix of few, long rows gives few workgroups, each with K / 256 dependent stages): TEAMS x 4 wavefronts; team
// t takes super-blocks t, TEAMS + t, ... of the same 32 rows, so TEAMS stages are in the pipes at once. The chain order is
// kept by team 0, which adds the terms of every super-block in ascending order: its own from registers, the other teams'
// from an LDS exchange buffer, one stage group behind (the group's barrier publishes them).
template <int NAL, int DEPTH, int TEAMS>
__global__ __launch_bounds__(256 * TEAMS) void q4k_mma_kernel(PairArgs args) {
    typedef __attribute__((address_space(3))) float lds_f32;
    constexpr uint32_t ACTS = mma_acts<NAL>(), CC = mma_code_copies<NAL>(), TOTAL = mma_copies<NAL>(), SLOT = mma_slot_bytes<NAL>();
    constexpr uint32_t PERW = (TOTAL + 3U) / 4U, FULL = TOTAL % 4U == 0 ? 4U : TOTAL % 4U;     // wavefronts 0 .. FULL - 1 of a team issue PERW copies
    constexpr uint32_t XTEAM = 4U * NAL * 64U;                                                  // floats one team exchanges per group
    static_assert(DEPTH >= 2 && DEPTH <= 8, "ring depth");
    static_assert(7U * PERW <= 63U, "vmcnt range");
    __shared__ __attribute__((aligned(16))) uint8_t ring_mem[DEPTH * TEAMS * SLOT];
    __shared__ float xbuf_mem[TEAMS > 1 ? 2U * (TEAMS - 1U) * XTEAM : 1U];
    lds_u8* const ring = (lds_u8*)ring_mem;
    lds_f32* const xbuf = (lds_f32*)xbuf_mem;
    if (args.skip_flag && (*args.skip_flag & args.skip_mask)) return;

    const PairMatrix& m = args.m[blockIdx.y];
    const uint32_t lane = threadIdx.x & 63U, j = lane & 31U, h = lane >> 5;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), p = wave & 3U, team = wave >> 2;
    const uint32_t row0 = blockIdx.x * kMmaRows, stages = args.blocks, groups = (stages + TEAMS - 1U) / TEAMS;
    const uint32_t my_groups = team < stages - (groups - 1U) * TEAMS ? groups : groups - 1U;   // groups in which this team has a super-block

    // ---- this wavefront's copies of a stage: copy c = 4k + p lands at slot + 1024 c
    const uint8_t* src[PERW];
    uint32_t step[PERW];
#pragma unroll
    for (uint32_t k = 0; k < PERW; ++k) {
        const uint32_t c = 4U * k + p;
        if (c < 5U) {                                           // weight pieces: 9 per row, rows back to back
            uint32_t s = 64U * c + lane;
            s = s < kMmaRows * 9U ? s : kMmaRows * 9U - 1U;     // the short fifth copy repeats the last piece into unused LDS
            const uint32_t r = s / 9U, piece = s - 9U * r;
            src[k] = m.w + static_cast<size_t>(row0 + r) * m.row_stride + 16U * piece;
            step[k] = 144U;
        } else if (c < 5U + CC) {                               // codes: 16 pieces per row, piece t at position (t + a) % 16
            const uint32_t s = 64U * (c - 5U) + lane, a = s >> 4, t = ((s & 15U) - a) & 15U;
            src[k] = reinterpret_cast<const uint8_t*>(args.img.codes_of(a < args.nacts ? a : 0U)) + 16U * t;
            step[k] = 256U;
        } else {                                                // table: per row [8 deltas][8 sums], four pieces
            const uint32_t a = lane >> 2, q = lane & 3U, row = a < ACTS && a < args.nacts ? a : 0U;
            src[k] = q < 2U ? reinterpret_cast<const uint8_t*>(args.img.deltas_of(row)) + 16U * q
                            : reinterpret_cast<const uint8_t*>(args.img.sums_of(row)) + 16U * (q - 2U);
            step[k] = 32U;
        }
        src[k] += static_cast<size_t>(step[k]) * team;
        step[k] *= TEAMS;
    }
    const auto start = [&](lds_u8* slot) {
#pragma unroll
        for (uint32_t k = 0; k < PERW; ++k) {
            const uint32_t c = 4U * k + p;
            if (c < TOTAL) {
                mma_copy16(src[k], slot + 1024U * c);
                src[k] += step[k];
            }
        }
    };

    MmaLane o;
    {
        const uint32_t ai = mma_slot_act<NAL>(j), c_base = 5120U + 256U * ai;
        o.head = 144U * j;
        o.quants = 144U * j + 16U + 32U * p + 16U * h;
        o.even = c_base + 16U * ((4U * p + h + ai) & 15U);
        o.odd = c_base + 16U * ((4U * p + 2U + h + ai) & 15U);
        // quad lane 0, 1: delta of sub-block 2p, 2p + 1; quad lane 2, 3: their code sums
        o.table = 5120U + 1024U * CC + 64U * h + 4U * (2U * p + (lane & 1U) + 4U * (lane & 2U));
        o.sum_lane = (lane & 2U) != 0;
    }

    float acc[NAL], own[NAL];
#pragma unroll
    for (int v = 0; v < NAL; ++v) { acc[v] = 0.0F; own[v] = 0.0F; }
    // team 0: the terms of group g (its own, then teams 1 .. of the super-blocks that exist), in super-block order
    const auto fold = [&](uint32_t g) {
#pragma unroll
        for (int v = 0; v < NAL; ++v) acc[v] = acc[v] + own[v];
#pragma unroll
        for (uint32_t t = 1; t < TEAMS; ++t) {
            if (g * TEAMS + t < stages) {
                const lds_f32* x = xbuf + ((g & 1U) * (TEAMS - 1U) + (t - 1U)) * XTEAM + p * NAL * 64U + lane;
#pragma unroll
                for (int v = 0; v < NAL; ++v) acc[v] = acc[v] + x[v * 64];
            }
        }
    };

    // ---- the ring of stage groups
    uint32_t issued = 0, issue_slot = 0, compute_slot = 0;
    const auto issue = [&]() {
        if (issued < my_groups) { start(ring + SLOT * (issue_slot * TEAMS + team)); ++issued; }
        issue_slot = issue_slot + 1U == DEPTH ? 0U : issue_slot + 1U;
    };
    for (uint32_t s = 0; s + 1U < DEPTH; ++s) issue();
    for (uint32_t g = 0; g < groups; ++g) {
        if (g < my_groups) {
            const uint32_t ahead = issued - 1U - g;              // this wavefront's stages started after its stage of group g
            if (p < FULL) mma_wait_n<PERW>(ahead);
            else mma_wait_n<PERW - 1U>(ahead);
        }
        mma_barrier();         // every copy of group g is in, the slots of group g - 1 are free, its exchanged terms are written
        issue();
        if (TEAMS > 1 && team == 0U && g > 0U) fold(g - 1U);
        if (g < my_groups) {
            const lds_u8* slot = ring + SLOT * (compute_slot * TEAMS + team);
            float term[NAL];
            switch (p) {
            case 0: mma_stage_terms<NAL, 0>(slot, o, term); break;
            case 1: mma_stage_terms<NAL, 1>(slot, o, term); break;
            case 2: mma_stage_terms<NAL, 2>(slot, o, term); break;
            default: mma_stage_terms<NAL, 3>(slot, o, term); break;
            }
            if (TEAMS == 1) {
#pragma unroll
                for (int v = 0; v < NAL; ++v) acc[v] = acc[v] + term[v];
            } else if (team == 0U) {
#pragma unroll
                for (int v = 0; v < NAL; ++v) own[v] = term[v];
            } else {
                lds_f32* x = xbuf + ((g & 1U) * (TEAMS - 1U) + (team - 1U)) * XTEAM + p * NAL * 64U + lane;
#pragma unroll
                for (int v = 0; v < NAL; ++v) x[v * 64] = term[v];
            }
        }
        compute_slot = compute_slot + 1U == DEPTH ? 0U : compute_slot + 1U;
    }

    // ---- value = (acc0 + acc1) + (acc2 + acc3) over team 0's four wavefronts; wavefront w stores result registers w, w + 4, ...
    __syncthreads();
    if (TEAMS > 1 && team == 0U) fold(groups - 1U);
    lds_f32* red = (lds_f32*)ring;
    if (team == 0U) {
#pragma unroll
        for (int v = 0; v < NAL; ++v) red[(p * NAL + v) * 64U + lane] = acc[v];
    }
    __syncthreads();
    if (team != 0U) return;
#pragma unroll
    for (uint32_t v = 0; v < NAL; ++v) {
        if ((v & 3U) != p) continue;
        const float r0 = red[(0U * NAL + v) * 64U + lane], r1 = red[(1U * NAL + v) * 64U + lane];
        const float r2 = red[(2U * NAL + v) * 64U + lane], r3 = red[(3U * NAL + v) * 64U + lane];
        const float left = r0 + r1, right = r2 + r3;
        const uint32_t a = 2U * v + h;
        if (a < args.nacts) m.out[static_cast<size_t>(a) * m.out_stride + row0 + j] = left + right;
    }
}

}  // namespace strix950
