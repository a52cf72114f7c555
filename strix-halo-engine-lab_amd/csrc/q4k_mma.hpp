// Q4_K x A8 rows against 3..32 activation rows at a time: the exact group dots come from the int8 matrix cores, the
// reference's fp32 chain stays on the vector ALU. The sweep below serves a dense matrix (q4k_mma_kernel) and the routed
// experts of larger batches (q4k_mma_moe.hpp: gate + up with the SwiGLU / A8 epilogue, and the down rows).
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
typedef __attribute__((address_space(3))) float lds_f32;

constexpr uint32_t kMmaRows = 32;
template <int NAL> constexpr uint32_t mma_acts() { return 2U * NAL; }                         // activation slots served (multiple of 4)
template <int NAL> constexpr uint32_t mma_code_copies() { return mma_acts<NAL>() / 4U; }      // 1 KiB = 4 rows x 256 codes
template <int NAL> constexpr uint32_t mma_table_copies() { return (mma_acts<NAL>() + 15U) / 16U; }   // 1 KiB = 16 rows x (8 deltas, 8 sums)
// NM matrices share the activation rows of a sweep (gate and up): 4.5 (5) KiB of weight pieces each
template <int NAL, int NM> constexpr uint32_t mma_copies() { return 5U * NM + mma_code_copies<NAL>() + mma_table_copies<NAL>(); }
template <int NAL, int NM> constexpr uint32_t mma_slot_bytes() { return 1024U * mma_copies<NAL, NM>(); }
template <int NAL, int NM, int DEPTH, int TEAMS> constexpr uint32_t mma_ring_bytes() { return DEPTH * TEAMS * mma_slot_bytes<NAL, NM>(); }
template <int NAL, int TEAMS> constexpr uint32_t mma_exchange_floats() { return TEAMS > 1 ? 2U * (TEAMS - 1U) * 4U * NAL * 64U : 1U; }

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
    static_assert(3 * N <= 63, "vmcnt range");
    switch (ahead) {
    case 0: mma_wait<0>(); break;
    case 1: mma_wait<N>(); break;
    case 2: mma_wait<2 * N>(); break;
    default: mma_wait<3 * N>(); break;
    }
}

// Activation row served by operand-A slot i (the inverse of "row a -> result register a / 2 of half a % 2"); slots past the
// served rows repeat earlier rows (their results are never read).
template <int NAL> __device__ __forceinline__ uint32_t mma_slot_act(uint32_t i) {
    const uint32_t v = 4U * (i >> 3) + (i & 3U), h = (i >> 2) & 1U;
    return (2U * v + h) % mma_acts<NAL>();
}

// Per-lane byte offsets into a ring slot (constant over the sweep); matrix m's weights sit 5120 m further on.
struct MmaLane {
    uint32_t head, quants, even, odd, table;
    bool sum_lane;
};

// One landed super-block: for each matrix the wavefront's two group dots of its 32 rows against every activation slot, then the
// lane's chain terms x[2P] + x[2P + 1] for its first nv activation rows. P is the wavefront's pair, a template argument so that
// the scale / min unpacking has constant shifts.
template <int NAL, int NM, int P>
__device__ __forceinline__ void mma_stage_terms(const lds_u8* slot, const MmaLane& o, uint32_t nv, float (&term)[NM][NAL]) {
    typedef const __attribute__((address_space(3))) u32x4 lds_u32x4;
    typedef const __attribute__((address_space(3))) int32_t lds_i32;
    const u32x4 a_even = *(lds_u32x4*)(slot + o.even), a_odd = *(lds_u32x4*)(slot + o.odd);
    u32x4 hd[NM], q[NM];
#pragma unroll
    for (int m = 0; m < NM; ++m) {
        hd[m] = *(lds_u32x4*)(slot + 5120U * m + o.head);
        q[m] = *(lds_u32x4*)(slot + 5120U * m + o.quants);
    }
    int32_t tab[NAL];
#pragma unroll
    for (int v = 0; v < NAL; ++v) tab[v] = *(lds_i32*)(slot + o.table + 128U * v);
    if (o.sum_lane) {                                       // quad lanes 2, 3 hold code sums: to float, once
#pragma unroll
        for (int v = 0; v < NAL; ++v) tab[v] = __builtin_bit_cast(int32_t, static_cast<float>(tab[v]));
    }
#pragma unroll
    for (int m = 0; m < NM; ++m) {
        const u32x4 lo = q[m] & 0x0f0f0f0fU, hi = (q[m] >> 4) & 0x0f0f0f0fU;
        const i32x16 zero = {0};
        const i32x16 dot_even = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, a_even), __builtin_bit_cast(i32x4, lo), zero, 0, 0, 0);
        const i32x16 dot_odd = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, a_odd), __builtin_bit_cast(i32x4, hi), zero, 0, 0, 0);
        uint32_t s0, m0, s1, m1;
        q4k_factors<2 * P>(hd[m], s0, m0);
        q4k_factors<2 * P + 1>(hd[m], s1, m1);
        const float d = half_bits_to_float(hd[m].x & 0xffffU), dm = half_bits_to_float(hd[m].x >> 16);
        const float D0 = d * static_cast<float>(s0), M0 = dm * static_cast<float>(m0);
        const float D1 = d * static_cast<float>(s1), M1 = dm * static_cast<float>(m1);
#pragma unroll
        for (int v = 0; v < NAL; ++v) {
            // the widest sweep skips the result registers past a short chunk, four at a time (straight-line code either way: a
            // loop exit here would turn the register arrays into indexed accesses)
            if (NAL > 8 && static_cast<uint32_t>(v & ~3) >= nv) continue;
            const float e0 = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(tab[v], 0x00, 0xF, 0xF, true));
            const float e1 = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(tab[v], 0x55, 0xF, 0xF, true));
            const float f0 = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(tab[v], 0xAA, 0xF, 0xF, true));
            const float f1 = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(tab[v], 0xFF, 0xF, 0xF, true));
            const float u0 = D0 * static_cast<float>(dot_even[v]), v0 = M0 * f0;
            const float u1 = D1 * static_cast<float>(dot_odd[v]), v1 = M1 * f1;
            const float x0 = e0 * (u0 - v0), x1 = e1 * (u1 - v1);
            term[m][v] = x0 + x1;
        }
    }
}

// The sweep of one 32-row tile (NM matrices' tiles that share the activation rows) over `stages` super-blocks against nacts <=
// 2 NAL activation rows: on return team 0's wavefront p holds in acc[m][v] pair accumulator p of (row j, activation row 2v + h).
// acts(a) names activation row a < nacts: .codes / .deltas / .sums point at its A8 image (K codes, K / 32 deltas and sums).
//
// TEAMS > 1 (a matrix of few, long rows gives few workgroups, each with K / 256 dependent stages): TEAMS x 4 wavefronts; team
// t takes super-blocks t, TEAMS + t, ... of the same 32 rows, so TEAMS stages are in the pipes at once. The chain order is
// kept by team 0, which adds the terms of every super-block in ascending order: its own from registers, the other teams'
// from an LDS exchange buffer, one stage group behind (the group's barrier publishes them).
// Every wavefront of the workgroup calls this; the ring is free again when it returns.
struct MmaActRow { const uint8_t *codes, *deltas, *sums; };
template <int NAL, int DEPTH, int TEAMS, int NM, class Acts>
__device__ __forceinline__ void mma_sweep(lds_u8* ring, lds_f32* xbuf, const uint8_t* const (&wrows)[NM], size_t row_stride, uint32_t stages,
                                          Acts acts, uint32_t nacts, float (&acc)[NM][NAL]) {
    constexpr uint32_t ACTS = mma_acts<NAL>(), CC = mma_code_copies<NAL>(), TOTAL = mma_copies<NAL, NM>(), SLOT = mma_slot_bytes<NAL, NM>();
    constexpr uint32_t PERW = (TOTAL + 3U) / 4U, FULL = TOTAL % 4U == 0 ? 4U : TOTAL % 4U;     // wavefronts 0 .. FULL - 1 of a team issue PERW copies
    constexpr uint32_t XTEAM = 4U * NAL * 64U;                                                  // floats one team exchanges per group
    static_assert(DEPTH >= 2 && DEPTH <= 4, "ring depth");
    static_assert(TEAMS == 1 || (NM == 1 && NAL <= 8), "stage teams serve one matrix, every result register");
    const uint32_t lane = threadIdx.x & 63U, j = lane & 31U, h = lane >> 5;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), p = wave & 3U, team = wave >> 2;
    const uint32_t groups = (stages + TEAMS - 1U) / TEAMS;
    const uint32_t my_groups = team < stages - (groups - 1U) * TEAMS ? groups : groups - 1U;   // groups in which this team has a super-block
    const uint32_t nv = (nacts + 1U) / 2U;

    // ---- this wavefront's copies of a stage: copy c = 4k + p lands at slot + 1024 c
    const uint8_t* src[PERW];
    uint32_t step[PERW];
#pragma unroll
    for (uint32_t k = 0; k < PERW; ++k) {
        const uint32_t c = 4U * k + p;
        if (c < 5U * NM) {                                      // weight pieces: 9 per row, rows back to back
            const uint32_t m = c / 5U;
            uint32_t s = 64U * (c - 5U * m) + lane;
            s = s < kMmaRows * 9U ? s : kMmaRows * 9U - 1U;     // the short fifth copy repeats the last piece into unused LDS
            const uint32_t r = s / 9U, piece = s - 9U * r;
            src[k] = wrows[m < NM ? m : 0] + static_cast<size_t>(r) * row_stride + 16U * piece;
            step[k] = 144U;
        } else if (c < 5U * NM + CC) {                          // codes: 16 pieces per row, piece t at position (t + a) % 16
            const uint32_t s = 64U * (c - 5U * NM) + lane, a = s >> 4, t = ((s & 15U) - a) & 15U;
            src[k] = acts(a < nacts ? a : 0U).codes + 16U * t;
            step[k] = 256U;
        } else {                                                // table: per row [8 deltas][8 sums], four pieces
            const uint32_t a = 16U * (c - 5U * NM - CC) + (lane >> 2), q = lane & 3U;
            const MmaActRow row = acts(a < ACTS && a < nacts ? a : 0U);
            src[k] = q < 2U ? row.deltas + 16U * q : row.sums + 16U * (q - 2U);
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
        const uint32_t ai = mma_slot_act<NAL>(j), c_base = 5120U * NM + 256U * ai;
        o.head = 144U * j;
        o.quants = 144U * j + 16U + 32U * p + 16U * h;
        o.even = c_base + 16U * ((4U * p + h + ai) & 15U);
        o.odd = c_base + 16U * ((4U * p + 2U + h + ai) & 15U);
        // quad lane 0, 1: delta of sub-block 2p, 2p + 1; quad lane 2, 3: their code sums
        o.table = 5120U * NM + 1024U * CC + 64U * h + 4U * (2U * p + (lane & 1U) + 4U * (lane & 2U));
        o.sum_lane = (lane & 2U) != 0;
    }

    float own[NAL];
#pragma unroll
    for (int v = 0; v < NAL; ++v) own[v] = 0.0F;
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int v = 0; v < NAL; ++v) acc[m][v] = 0.0F;
    // team 0: the terms of group g (its own, then teams 1 .. of the super-blocks that exist), in super-block order
    const auto fold = [&](uint32_t g) {
#pragma unroll
        for (int v = 0; v < NAL; ++v) acc[0][v] = acc[0][v] + own[v];
#pragma unroll
        for (uint32_t t = 1; t < TEAMS; ++t) {
            if (g * TEAMS + t < stages) {
                const lds_f32* x = xbuf + ((g & 1U) * (TEAMS - 1U) + (t - 1U)) * XTEAM + p * NAL * 64U + lane;
#pragma unroll
                for (int v = 0; v < NAL; ++v) acc[0][v] = acc[0][v] + x[v * 64];
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
            float term[NM][NAL];
            switch (p) {
            case 0: mma_stage_terms<NAL, NM, 0>(slot, o, nv, term); break;
            case 1: mma_stage_terms<NAL, NM, 1>(slot, o, nv, term); break;
            case 2: mma_stage_terms<NAL, NM, 2>(slot, o, nv, term); break;
            default: mma_stage_terms<NAL, NM, 3>(slot, o, nv, term); break;
            }
            if (TEAMS == 1) {
#pragma unroll
                for (int m = 0; m < NM; ++m)
#pragma unroll
                    for (int v = 0; v < NAL; ++v) {
                        if (NAL > 8 && static_cast<uint32_t>(v & ~3) >= nv) continue;
                        acc[m][v] = acc[m][v] + term[m][v];
                    }
            } else if (team == 0U) {
#pragma unroll
                for (int v = 0; v < NAL; ++v) own[v] = term[0][v];
            } else {
                lds_f32* x = xbuf + ((g & 1U) * (TEAMS - 1U) + (team - 1U)) * XTEAM + p * NAL * 64U + lane;
#pragma unroll
                for (int v = 0; v < NAL; ++v) x[v * 64] = term[0][v];
            }
        }
        compute_slot = compute_slot + 1U == DEPTH ? 0U : compute_slot + 1U;
    }
    __syncthreads();           // no copy in flight (the last wait was for all), every LDS read of the ring is done
    if (TEAMS > 1 && team == 0U) fold(groups - 1U);
}

// value = (acc0 + acc1) + (acc2 + acc3) over team 0's four wavefronts, through `red` (4 NM NAL 64 floats, may be the ring):
// wavefront w of team 0 receives the values of result registers v = w, w + 4, ... and hands (v, values of the NM matrices) to
// emit. Every wavefront of the workgroup calls this; `red` is free again when it returns.
template <int NAL, int NM, class Emit>
__device__ __forceinline__ void mma_reduce(lds_f32* red, const float (&acc)[NM][NAL], uint32_t nacts, Emit emit) {
    const uint32_t lane = threadIdx.x & 63U;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), p = wave & 3U, team = wave >> 2;
    const uint32_t nv = (nacts + 1U) / 2U;
    if (team == 0U) {
#pragma unroll
        for (int m = 0; m < NM; ++m)
#pragma unroll
            for (int v = 0; v < NAL; ++v) red[((m * 4U + p) * NAL + v) * 64U + lane] = acc[m][v];
    }
    __syncthreads();
    if (team == 0U) {
#pragma unroll
        for (uint32_t v = 0; v < NAL; ++v) {
            if ((v & 3U) != p || v >= nv) continue;
            float value[NM];
#pragma unroll
            for (int m = 0; m < NM; ++m) {
                const float r0 = red[((m * 4U + 0U) * NAL + v) * 64U + lane], r1 = red[((m * 4U + 1U) * NAL + v) * 64U + lane];
                const float r2 = red[((m * 4U + 2U) * NAL + v) * 64U + lane], r3 = red[((m * 4U + 3U) * NAL + v) * 64U + lane];
                const float left = r0 + r1, right = r2 + r3;
                value[m] = left + right;
            }
            emit(v, value);
        }
    }
    __syncthreads();
}

// ---- a dense matrix (or two that share their activation rows), rows of raw dots out
template <int NAL, int DEPTH, int TEAMS>
__global__ __launch_bounds__(256 * TEAMS) void q4k_mma_kernel(PairArgs args) {
    __shared__ __attribute__((aligned(16))) uint8_t ring_mem[mma_ring_bytes<NAL, 1, DEPTH, TEAMS>()];
    __shared__ float xbuf_mem[mma_exchange_floats<NAL, TEAMS>()];
    if (args.skip_flag && (*args.skip_flag & args.skip_mask)) return;
    const PairMatrix& m = args.m[blockIdx.y];
    const uint32_t lane = threadIdx.x & 63U, row0 = blockIdx.x * kMmaRows;
    const uint8_t* const wrows[1] = {m.w + static_cast<size_t>(row0) * m.row_stride};
    const A8Image& img = args.img;
    const auto acts = [&](uint32_t a) {
        return MmaActRow{reinterpret_cast<const uint8_t*>(img.codes_of(a)), reinterpret_cast<const uint8_t*>(img.deltas_of(a)),
                         reinterpret_cast<const uint8_t*>(img.sums_of(a))};
    };
    float acc[1][NAL];
    mma_sweep<NAL, DEPTH, TEAMS, 1>((lds_u8*)ring_mem, (lds_f32*)xbuf_mem, wrows, m.row_stride, args.blocks, acts, args.nacts, acc);
    mma_reduce<NAL, 1>((lds_f32*)ring_mem, acc, args.nacts, [&](uint32_t v, const float (&value)[1]) {
        const uint32_t a = 2U * v + (lane >> 5);
        if (a < args.nacts) m.out[static_cast<size_t>(a) * m.out_stride + row0 + (lane & 31U)] = value[0];
    });
}

}  // namespace strix950
