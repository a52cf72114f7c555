// Down rows in the formats of the reference's host executor: Q8_0 and Q5_1 blocks of 32 weights against the A8 image of h
// (src/cpu/core/routed_expert.cpp:110-144, "down (Q5_1 | Q8_0, groups of 32, chain j 0..3 owns groups g = 4c + j, c
// ascending)", src/cpu/core/routed_expert.hpp:13). Per group: an exact int32 dot, first = d * float(dot),
// Q5_1: combined = first + (m * float(sum of the group's codes)), chain[g % 4] += delta_g * combined; the row's value is
// (chain0 + chain1) + (chain2 + chain3).
//
// The four chains of a row are independent, so a wavefront holds 16 output rows with lane = (row, chain): a lane walks
// its chain's groups in ascending order and two quad exchanges form the value, bit for bit the sequential result. A
// 256-thread workgroup covers 64 output rows of one plan item (an expert and up to `split` of its assignments); every
// weight block a lane loads is used for up to four assignments before the next one is fetched.
//
// Block addresses. Q8_0 blocks are 34 bytes, so a row's blocks alternate between 4-byte and 2-byte alignment; the chain
// index fixes which (g = 4c + j is odd exactly when j is). A lane reads nine aligned words: for even j the words from the
// block's start (d in the low half of the first, every code word straddling two of them), for odd j the eight words from the
// first code and the word before them (d in its high half). Q5_1 blocks are 24 bytes (fp16 d, fp16 m, 32 fifth bits, 16
// bytes of nibbles; weight k is nibble k % 16 of the low (k < 16) or high halves plus bit k of the fifth-bit word) and
// always 8-byte aligned.
#pragma once
#include "device_math.hpp"
#include "q4k_rows.hpp"

namespace strix950 {

constexpr uint32_t kDownGroupsRows = 64;       // output rows per workgroup (4 waves x 16)
constexpr uint32_t kDownGroupsAssignments = 4; // assignments per weight pass

// FMT 0: Q8_0, FMT 1: Q5_1. Loads the lane's block and returns d, m and the eight words of signed / 5-bit codes in the
// order of the activation codes.
template <int FMT>
__device__ __forceinline__ void load_group_block(const uint8_t* block, uint32_t odd, float& d, float& m, uint32_t (&q)[8]) {
    typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
    typedef uint32_t u32x2_a4 __attribute__((ext_vector_type(2), aligned(4)));
    if (FMT == 0) {
        const uint8_t* first = block + 2U * odd;                              // odd: the first code, even: the block's start
        const u32x4_a4 a = *reinterpret_cast<const u32x4_a4*>(first), b = *reinterpret_cast<const u32x4_a4*>(first + 16);
        const uint32_t c = *reinterpret_cast<const uint32_t*>(odd ? first - 4 : first + 32);
        const uint32_t seq[9] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w, c};
        const uint32_t straddle = odd ? 0U : 2U;
#pragma unroll
        for (int i = 0; i < 8; ++i) q[i] = __builtin_amdgcn_alignbyte(i == 7 && odd ? seq[7] : seq[i + 1], seq[i], straddle);
        d = half_bits_to_float(odd ? c >> 16 : a.x & 0xffffU);
        m = 0.0F;
    } else {
        const u32x2_a4 head = *reinterpret_cast<const u32x2_a4*>(block);
        const u32x4_a4 nib = *reinterpret_cast<const u32x4_a4*>(block + 8);
        d = half_bits_to_float(head.x & 0xffffU);
        m = half_bits_to_float(head.x >> 16);
        const uint32_t fifth = head.y, n[4] = {nib.x, nib.y, nib.z, nib.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            // four bits of the fifth-bit word -> bit 4 of four bytes: the product places bit b at 8 b (the shifted copies
            // of a 4-bit value do not overlap, so nothing carries)
            const uint32_t lo5 = (((fifth >> (4 * i)) & 15U) * 0x00204081U & 0x01010101U) << 4;
            const uint32_t hi5 = (((fifth >> (16 + 4 * i)) & 15U) * 0x00204081U & 0x01010101U) << 4;
            q[i] = (n[i] & 0x0f0f0f0fU) | lo5;
            q[4 + i] = ((n[i] >> 4) & 0x0f0f0f0fU) | hi5;
        }
    }
}

template <int FMT>
__global__ __launch_bounds__(256) void down_groups_kernel(mi355_moe_weights w, RowsK r, uint32_t assignments,
                                                          uint32_t items_at, uint32_t order_at) {
    typedef uint32_t u32x4_g __attribute__((ext_vector_type(4)));
    const WorkItem item = work_item(w, r, items_at, blockIdx.y);
    const uint32_t e = item.e, begin = item.begin, end = item.end;
    if (begin == end) return;
    if (*r.job_status & MI355_STATUS_NONFINITE_PROJECTION) return;
    const uint32_t lane = threadIdx.x & 63U, wave = threadIdx.x >> 6, j = lane & 3U, odd = j & 1U;
    const uint32_t o = blockIdx.x * kDownGroupsRows + 16U * wave + (lane >> 2);
    const uint32_t groups = w.ffn / 32U, per_chain = groups / 4U;
    constexpr uint32_t kBlock = FMT == 0 ? 34U : 24U;
    const uint8_t* wrow = w.down + static_cast<size_t>(e) * w.down_expert_stride + static_cast<size_t>(o) * w.down_row_stride + kBlock * j;
    for (uint32_t c0 = begin; c0 < end; c0 += kDownGroupsAssignments) {
        const uint32_t na = end - c0 < kDownGroupsAssignments ? end - c0 : kDownGroupsAssignments;
        uint32_t src[kDownGroupsAssignments];
        float chain[kDownGroupsAssignments];
        const int8_t* h_codes[kDownGroupsAssignments];
        const float* h_deltas[kDownGroupsAssignments];
        const int32_t* h_sums[kDownGroupsAssignments];
#pragma unroll
        for (uint32_t a = 0; a < kDownGroupsAssignments; ++a) {
            src[a] = ordered(r, order_at, c0 + (a < na ? a : na - 1U));
            chain[a] = 0.0F;
            h_codes[a] = r.h.codes_of(src[a]);
            h_deltas[a] = r.h.deltas_of(src[a]);
            h_sums[a] = r.h.sums_of(src[a]);
        }
#pragma unroll 2
        for (uint32_t c = 0; c < per_chain; ++c) {
            const uint32_t g = 4U * c + j;
            float d, m;
            uint32_t q[8];
            load_group_block<FMT>(wrow + static_cast<size_t>(c) * (4U * kBlock), odd, d, m, q);
#pragma unroll
            for (uint32_t a = 0; a < kDownGroupsAssignments; ++a) {
                if (a < na) {                                     // uniform over the workgroup
                    const u32x4_g* codes = reinterpret_cast<const u32x4_g*>(h_codes[a] + 32U * g);
                    const u32x4_g c_lo = codes[0], c_hi = codes[1];
                    const uint32_t cw[8] = {c_lo.x, c_lo.y, c_lo.z, c_lo.w, c_hi.x, c_hi.y, c_hi.z, c_hi.w};
                    int dot = 0;
#pragma unroll
                    for (int i = 0; i < 8; ++i) dot = __builtin_amdgcn_sdot4(static_cast<int>(q[i]), static_cast<int>(cw[i]), dot, false);
                    const float first = d * static_cast<float>(dot);
                    float combined = first;
                    if (FMT == 1) combined = first + (m * static_cast<float>(h_sums[a][g]));
                    chain[a] = chain[a] + (h_deltas[a][g] * combined);
                }
            }
        }
#pragma unroll
        for (uint32_t a = 0; a < kDownGroupsAssignments; ++a) {
            if (a < na) {
                float v = chain[a];
                v = v + xor1_f(v);          // chain0 + chain1 | chain2 + chain3
                v = v + xor2_f(v);          // (chain0 + chain1) + (chain2 + chain3)
                if (j == 0) r.rawdots_of(src[a], w.hidden)[o] = v;
            }
        }
    }
}

// ---- the same rows streamed through a copy ring ------------------------------------------------------------------------
// Q5_1 only: the Q8_0 rows gain nothing from it (their 34-byte blocks come out of LDS as nine 32-bit reads each: 27.2 us against
// 26.9 us with the direct loads above, config 3 with 8 rows), the Q5_1 rows 24.6 -> 19.1 us.
// A stage is 8 groups (one 256-value super-block of K) of the wave's 16 rows - 192 consecutive bytes per row, 16-byte pieces copied global -> LDS by global_load_lds_dwordx4 - plus the 256 codes and the 8 deltas / sums of the same 8
// groups of up to four activation rows (a plain load of those inside the loop would make the wave wait for every copy issued
// before it); DEPTH slots per wave, waits counted. Needs ffn % 256 == 0 and 16-byte aligned rows (the launcher checks);
// the arithmetic and its order are those of down_groups_kernel above.
constexpr uint32_t kGroupStage = 8;            // groups per stage
constexpr uint32_t kQ51Block = 24;
constexpr uint32_t group_row_pieces() { return kGroupStage * kQ51Block / 16U; }                                 // 12
constexpr uint32_t group_weight_copies() { return (16U * group_row_pieces() + 63U) / 64U; }                       // 3
constexpr uint32_t group_slot_bytes() { return 1024U * (group_weight_copies() + 2U); }             // + codes, + deltas / sums

// Block at `block` (LDS, 8-byte aligned): d, m and the eight code words, as load_group_block<1> gives them.
__device__ __forceinline__ void load_q51_block_lds(const lds_u8* block, float& d, float& m, uint32_t (&q)[8]) {
    typedef const __attribute__((address_space(3))) uint32_t lds_u32;
    lds_u32* w = (lds_u32*)block;
    const uint32_t head = w[0], fifth = w[1], n[4] = {w[2], w[3], w[4], w[5]};
    d = half_bits_to_float(head & 0xffffU);
    m = half_bits_to_float(head >> 16);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t lo5 = (((fifth >> (4 * i)) & 15U) * 0x00204081U & 0x01010101U) << 4;
        const uint32_t hi5 = (((fifth >> (16 + 4 * i)) & 15U) * 0x00204081U & 0x01010101U) << 4;
        q[i] = (n[i] & 0x0f0f0f0fU) | lo5;
        q[4 + i] = ((n[i] >> 4) & 0x0f0f0f0fU) | hi5;
    }
}

#define STRIX_GROUP_SLOTS(DEPTH)                                                                                         \
    __shared__ __attribute__((aligned(16))) uint8_t grp0[4][group_slot_bytes()];                                     \
    __shared__ __attribute__((aligned(16))) uint8_t grp1[4][group_slot_bytes()];                                     \
    __shared__ __attribute__((aligned(16))) uint8_t grp2[DEPTH > 2 ? 4 : 1][DEPTH > 2 ? group_slot_bytes() : 16];    \
    __shared__ __attribute__((aligned(16))) uint8_t grp3[DEPTH > 3 ? 4 : 1][DEPTH > 3 ? group_slot_bytes() : 16];    \
    lds_u8* const grp_ring[4] = {(lds_u8*)grp0[wave], (lds_u8*)grp1[wave], (lds_u8*)grp2[DEPTH > 2 ? wave : 0], (lds_u8*)grp3[DEPTH > 3 ? wave : 0]};

template <int DEPTH>
__global__ __launch_bounds__(256) void down_q51_ring_kernel(mi355_moe_weights w, RowsK r, uint32_t assignments,
                                                               uint32_t items_at, uint32_t order_at) {
    typedef const __attribute__((address_space(3))) u32x4 lds_u32x4;
    typedef const __attribute__((address_space(3))) float lds_f32c;
    typedef const __attribute__((address_space(3))) int32_t lds_i32c;
    constexpr uint32_t kBlock = kQ51Block, RP = group_row_pieces(), WC = group_weight_copies(), PER = WC + 2U;
    constexpr uint32_t ROWB = kGroupStage * kBlock, CODES_AT = 1024U * WC, TABLE_AT = CODES_AT + 1024U;
    const uint32_t wave = threadIdx.x >> 6;
    STRIX_GROUP_SLOTS(DEPTH)
    const WorkItem item = work_item(w, r, items_at, blockIdx.y);
    const uint32_t e = item.e, begin = item.begin, end = item.end;
    if (begin == end) return;
    if (*r.job_status & MI355_STATUS_NONFINITE_PROJECTION) return;
    const uint32_t lane = threadIdx.x & 63U, j = lane & 3U, rr = lane >> 2;
    const uint32_t o0 = blockIdx.x * kDownGroupsRows + 16U * wave, o = o0 + rr;
    const uint32_t stages = w.ffn / 256U;
    const uint8_t* rows = w.down + static_cast<size_t>(e) * w.down_expert_stride + static_cast<size_t>(o0) * w.down_row_stride;
    // the lane's pieces of a stage: piece index i * 64 + lane = row * RP + piece of the row's 8-group segment
    const uint8_t* wsrc0[WC];
#pragma unroll
    for (uint32_t i = 0; i < WC; ++i) {
        uint32_t k = i * 64U + lane;
        k = k < 16U * RP ? k : 16U * RP - 1U;                  // padding lanes repeat the last piece into unused LDS
        const uint32_t row = k / RP, piece = k - RP * row;
        wsrc0[i] = rows + static_cast<size_t>(row) * w.down_row_stride + 16U * piece;
    }
    for (uint32_t c0 = begin; c0 < end; c0 += kDownGroupsAssignments) {
        const uint32_t na = end - c0 < kDownGroupsAssignments ? end - c0 : kDownGroupsAssignments;
        uint32_t src[kDownGroupsAssignments];
        float chain[kDownGroupsAssignments];
#pragma unroll
        for (uint32_t a = 0; a < kDownGroupsAssignments; ++a) {
            src[a] = ordered(r, order_at, c0 + (a < na ? a : na - 1U));
            chain[a] = 0.0F;
        }
        // codes copy: lane = (activation row lane / 16, piece lane % 16) of the stage's 256 codes
        const uint8_t* csrc = reinterpret_cast<const uint8_t*>(r.h.codes_of(ordered(r, order_at, c0 + ((lane >> 4) < na ? (lane >> 4) : na - 1U)))) + 16U * (lane & 15U);
        // table copy: per activation row [8 deltas][8 sums]; lane & 15 = (row, piece): pieces 0, 1 the deltas, 2, 3 the sums
        const uint8_t* tsrc;
        {
            const uint32_t ta = (lane >> 2) & 3U, tq = lane & 3U, ti = ordered(r, order_at, c0 + (ta < na ? ta : na - 1U));
            tsrc = tq < 2U ? reinterpret_cast<const uint8_t*>(r.h.deltas_of(ti)) + 16U * tq : reinterpret_cast<const uint8_t*>(r.h.sums_of(ti)) + 16U * (tq - 2U);
        }
        const uint8_t* wsrc[WC];
#pragma unroll
        for (uint32_t i = 0; i < WC; ++i) wsrc[i] = wsrc0[i];
        const auto start = [&](lds_u8* slot) {
#pragma unroll
            for (uint32_t i = 0; i < WC; ++i) {
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)wsrc[i],
                                                 (__attribute__((address_space(3))) void*)(slot + 1024U * i), 16, 0, 0);
                wsrc[i] += ROWB;
            }
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)csrc,
                                             (__attribute__((address_space(3))) void*)(slot + CODES_AT), 16, 0, 0);
            csrc += 256;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)tsrc,
                                             (__attribute__((address_space(3))) void*)(slot + TABLE_AT), 16, 0, 0);
            tsrc += 32;
        };
#pragma unroll
        for (int s = 0; s < DEPTH - 1; ++s)
            if (static_cast<uint32_t>(s) < stages) start(grp_ring[s]);
        for (uint32_t b0 = 0; b0 < stages; b0 += DEPTH) {
#pragma unroll
            for (int s = 0; s < DEPTH; ++s) {
                const uint32_t b = b0 + s;
                if (b < stages) {
                    const uint32_t last = b + DEPTH - 1U < stages ? b + DEPTH - 1U : stages;
                    wait_stages_ahead<PER>(last - 1U - b);
                    if (b + DEPTH - 1U < stages) start(grp_ring[(s + DEPTH - 1) % DEPTH]);
                    const lds_u8* slot = grp_ring[s];
#pragma unroll
                    for (uint32_t c = 0; c < kGroupStage / 4U; ++c) {
                        const uint32_t gl = 4U * c + j;                                 // the lane's group inside the stage
                        float d, m;
                        uint32_t q[8];
                        load_q51_block_lds(slot + rr * ROWB + gl * kBlock, d, m, q);
#pragma unroll
                        for (uint32_t a = 0; a < kDownGroupsAssignments; ++a) {
                            if (a < na) {                                     // uniform over the workgroup
                                lds_u32x4* codes = (lds_u32x4*)(slot + CODES_AT + 256U * a + 32U * gl);
                                const u32x4 c_lo = codes[0], c_hi = codes[1];
                                const uint32_t cw[8] = {c_lo.x, c_lo.y, c_lo.z, c_lo.w, c_hi.x, c_hi.y, c_hi.z, c_hi.w};
                                int dot = 0;
#pragma unroll
                                for (int i = 0; i < 8; ++i) dot = __builtin_amdgcn_sdot4(static_cast<int>(q[i]), static_cast<int>(cw[i]), dot, false);
                                const float first = d * static_cast<float>(dot);
                                const float combined = first + (m * static_cast<float>(*(lds_i32c*)(slot + TABLE_AT + 64U * a + 32U + 4U * gl)));
                                chain[a] = chain[a] + (*(lds_f32c*)(slot + TABLE_AT + 64U * a + 4U * gl) * combined);
                            }
                        }
                    }
                }
            }
        }
#pragma unroll
        for (uint32_t a = 0; a < kDownGroupsAssignments; ++a) {
            if (a < na) {
                float v = chain[a];
                v = v + xor1_f(v);          // chain0 + chain1 | chain2 + chain3
                v = v + xor2_f(v);          // (chain0 + chain1) + (chain2 + chain3)
                if (j == 0) r.rawdots_of(src[a], w.hidden)[o] = v;
            }
        }
    }
}

}  // namespace strix950
