// Q4_K x A8 rows for the smallest decode batches (one or two tokens): a wavefront evaluates 16 weight rows against ONE
// activation row, lane = (row r, pair p) with p in the low two bits. A lane owns the reference's pair accumulator p of its
// row (sub-blocks 2p and 2p + 1 of every super-block); value = (acc0 + acc1) + (acc2 + acc3) by two quad exchanges.
//
// Why a third sweep: with one token a layer touches top_k experts, and the row-per-lane sweep (q4k_rows.hpp, 64 rows per
// wavefront) then has a few hundred wavefronts whose instruction streams - the whole of K, four pairs per lane - are the
// launch's critical path. The four pair accumulators of a row are independent chains, so this layout has four times the
// wavefronts, each with a quarter of the instructions, and the same sums bit for bit.
//
// A stage is one super-block of the wave's 16 rows (2,304 bytes = 144 pieces of 16 bytes, three global_load_lds of which
// the third is partly padding) plus the 256 codes of the activation row's super-block; DEPTH slots of 4 KB form the ring.
// Group deltas / sums sit one group per lane as in q4k_rows.hpp; the lane's two groups are fetched with ds_bpermute.
// Reference arithmetic: src/cpu/core/routed_expert.cpp:73-108 == src/moe_q4k_a8_contract.cpp:126-140.
#pragma once
#include "q4k_rows.hpp"

namespace strix950 {

constexpr uint32_t kQuadRows = 16;
constexpr uint32_t kQuadSlotBytes = 4096;          // [0, 3072): weights (144 pieces + padding), [3072, 4096): codes (256 bytes + padding)
constexpr uint32_t kQuadCopies = 4;                // copy instructions per stage

// PIECES = 16-byte pieces of one row's block: 9 (Q4_K, 144 bytes) or 11 (Q5_K, 176 bytes); 16 rows are 144 / 176 pieces, three
// copy instructions either way (the third partly padding).
template <uint32_t PIECES>
struct QuadSourceT {
    const uint8_t* piece[3];
    const uint8_t* act_piece;
    // row_ptr(r) = first byte of weight row r (0..15); codes = the activation row's codes
    template <class RowPtr>
    __device__ __forceinline__ void init(RowPtr row_ptr, const int8_t* codes) {
        const uint32_t lane = threadIdx.x & 63U;
#pragma unroll
        for (uint32_t i = 0; i < 3U; ++i) {
            uint32_t j = i * 64U + lane;
            j = j < kQuadRows * PIECES ? j : kQuadRows * PIECES - 1U;      // padding lanes repeat the last piece into unused LDS
            const uint32_t r = j / PIECES, c = j - PIECES * r;
            piece[i] = row_ptr(r) + 16U * c;
        }
        act_piece = reinterpret_cast<const uint8_t*>(codes) + 16U * (lane & 15U);
    }
    __device__ __forceinline__ void start(lds_u8* slot) {
#pragma unroll
        for (uint32_t i = 0; i < 3U; ++i) {
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)piece[i],
                                             (__attribute__((address_space(3))) void*)(slot + 1024U * i), 16, 0, 0);
            piece[i] += 16U * PIECES;
        }
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)act_piece,
                                         (__attribute__((address_space(3))) void*)(slot + 3072U), 16, 0, 0);
        act_piece += 256;
    }
};
typedef QuadSourceT<9> QuadSource;

// The pair term of a super-block from its header words and the two integer dots (sub-blocks 2p, 2p + 1):
// x_j = delta_j * (d * sc_j * float(dot_j) - dmin * m_j * float(sum_j)), returned as x_2p + x_(2p+1). e0 / e1: the group
// deltas, f0 / f1: the group sums as floats. Reference: src/cpu/core/routed_expert.cpp:87-104 (the same for Q4_K and Q5_K).
__device__ __forceinline__ float quad_pair_term(const u32x4& hd, uint32_t p, int dot0, int dot1, float e0, float e1, float f0, float f1) {
    // 6-bit scale / min of sub-blocks 2p, 2p + 1 (src/cpu/core/routed_expert.cpp:65-71); branch-free choice between the two
    // packings (pairs 0, 1: 6 low bits; pairs 2, 3: 4 + 2 split bits)
    const uint32_t sh0 = 16U * (p & 1U), sh1 = sh0 + 8U;
    const uint32_t fa0 = (hd.y >> sh0) & 255U, fb0 = (hd.z >> sh0) & 255U, fc0 = (hd.w >> sh0) & 255U;
    const uint32_t fa1 = (hd.y >> sh1) & 255U, fb1 = (hd.z >> sh1) & 255U, fc1 = (hd.w >> sh1) & 255U;
    const uint32_t lowmask = 0U - static_cast<uint32_t>(p < 2U);
    const auto pick = [lowmask](uint32_t lo6, uint32_t split) { return split ^ ((lo6 ^ split) & lowmask); };
    const uint32_t s0 = pick(fa0 & 63U, (fc0 & 15U) | ((fa0 >> 6) << 4)), m0 = pick(fb0 & 63U, (fc0 >> 4) | ((fb0 >> 6) << 4));
    const uint32_t s1 = pick(fa1 & 63U, (fc1 & 15U) | ((fa1 >> 6) << 4)), m1 = pick(fb1 & 63U, (fc1 >> 4) | ((fb1 >> 6) << 4));
    const float d = half_bits_to_float(hd.x & 0xffffU), dm = half_bits_to_float(hd.x >> 16);
    const float D0 = d * static_cast<float>(s0), M0 = dm * static_cast<float>(m0);
    const float D1 = d * static_cast<float>(s1), M1 = dm * static_cast<float>(m1);
    const float u0 = D0 * static_cast<float>(dot0), v0 = M0 * f0;
    const float u1 = D1 * static_cast<float>(dot1), v1 = M1 * f1;
    const float x0 = e0 * (u0 - v0), x1 = e1 * (u1 - v1);
    return x0 + x1;
}

// One super-block (index kb along K): the lane's pair of its row. vd / vf: the activation row's group deltas / sums,
// group 8 (kb % 8) + j in lane 8 (kb % 8) + j.
__device__ __forceinline__ void quad_block_compute(const lds_u8* slot, uint32_t kb, float vd, float vf, float& acc) {
    typedef const __attribute__((address_space(3))) u32x4 lds_u32x4;
    const uint32_t lane = threadIdx.x & 63U, p = lane & 3U, r = lane >> 2;
    lds_u32x4* blk = (lds_u32x4*)(slot + r * 144U);
    const u32x4 hd = blk[0], q0 = blk[1U + 2U * p], q1 = blk[2U + 2U * p];
    lds_u32x4* c = (lds_u32x4*)(slot + 3072U + 64U * p);
    const u32x4 c0 = c[0], c1 = c[1], c2 = c[2], c3 = c[3];
    const uint32_t w[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
    const uint32_t cw[16] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w, c2.x, c2.y, c2.z, c2.w, c3.x, c3.y, c3.z, c3.w};
    int dot0 = 0, dot1 = 0;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        dot0 = __builtin_amdgcn_sdot4(static_cast<int>(w[k] & 0x0f0f0f0fU), static_cast<int>(cw[k]), dot0, false);
        dot1 = __builtin_amdgcn_sdot4(static_cast<int>((w[k] >> 4) & 0x0f0f0f0fU), static_cast<int>(cw[8 + k]), dot1, false);
    }
    const int from = static_cast<int>((kb & 7U) * 8U + 2U * p);
    const float e0 = __shfl(vd, from), e1 = __shfl(vd, from + 1), f0 = __shfl(vf, from), f1 = __shfl(vf, from + 1);
    acc = acc + quad_pair_term(hd, p, dot0, dot1, e0, e1, f0, f1);
}

// The same for a Q5_K super-block (176 bytes: header, 32 fifth-bit bytes - bit j of byte k belongs to element k of sub-block j -,
// 128 nibble bytes; q = nibble | fifth bit << 4; src/cpu/core/routed_expert.cpp:73-108 with Q5K).
__device__ __forceinline__ void quad_block_compute_q5k(const lds_u8* slot, uint32_t kb, float vd, float vf, float& acc) {
    typedef const __attribute__((address_space(3))) u32x4 lds_u32x4;
    const uint32_t lane = threadIdx.x & 63U, p = lane & 3U, r = lane >> 2;
    lds_u32x4* blk = (lds_u32x4*)(slot + r * 176U);
    const u32x4 hd = blk[0], h0 = blk[1], h1 = blk[2], q0 = blk[3U + 2U * p], q1 = blk[4U + 2U * p];
    lds_u32x4* c = (lds_u32x4*)(slot + 3072U + 64U * p);
    const u32x4 c0 = c[0], c1 = c[1], c2 = c[2], c3 = c[3];
    const uint32_t qs[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
    const uint32_t qh[8] = {h0.x, h0.y, h0.z, h0.w, h1.x, h1.y, h1.z, h1.w};
    const uint32_t cw[16] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w, c2.x, c2.y, c2.z, c2.w, c3.x, c3.y, c3.z, c3.w};
    int dot0 = 0, dot1 = 0;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const uint32_t fifth = qh[k] >> (2U * p);                        // bit 0 of every byte: sub-block 2p, bit 1: 2p + 1
        const uint32_t lo = (qs[k] & 0x0f0f0f0fU) | ((fifth & 0x01010101U) << 4);
        const uint32_t hi = ((qs[k] >> 4) & 0x0f0f0f0fU) | ((fifth & 0x02020202U) << 3);
        dot0 = __builtin_amdgcn_sdot4(static_cast<int>(lo), static_cast<int>(cw[k]), dot0, false);
        dot1 = __builtin_amdgcn_sdot4(static_cast<int>(hi), static_cast<int>(cw[8 + k]), dot1, false);
    }
    const int from = static_cast<int>((kb & 7U) * 8U + 2U * p);
    const float e0 = __shfl(vd, from), e1 = __shfl(vd, from + 1), f0 = __shfl(vf, from), f1 = __shfl(vf, from + 1);
    acc = acc + quad_pair_term(hd, p, dot0, dot1, e0, e1, f0, f1);
}

// Whole sweep of the wave's 16 rows against activation row `row` of `img`; every lane of a quad returns the row's value.
template <int DEPTH, bool Q5K = false>
__device__ __forceinline__ float sweep_quads(lds_u8* const (&slots)[DEPTH], QuadSourceT<Q5K ? 11U : 9U> source, uint32_t blocks, const A8Image& img, uint32_t row) {
    const uint32_t lane = threadIdx.x & 63U, groups = img.width / 32U;
    const float* deltas = img.deltas_of(row);
    const int32_t* sums = img.sums_of(row);
    float acc = 0.0F, vd = 0.0F, vf = 0.0F;
#pragma unroll
    for (int s = 0; s < DEPTH - 1; ++s)
        if (static_cast<uint32_t>(s) < blocks) source.start(slots[s]);
    for (uint32_t b0 = 0; b0 < blocks; b0 += DEPTH) {
#pragma unroll
        for (int s = 0; s < DEPTH; ++s) {
            const uint32_t b = b0 + s;
            if (b < blocks) {
                if ((b & 7U) == 0) {           // refill the per-lane group deltas / sums: groups 8 b .. 8 b + 63
                    const uint32_t g = b * 8U + lane;
                    vd = g < groups ? deltas[g] : 0.0F;
                    vf = g < groups ? static_cast<float>(sums[g]) : 0.0F;
                }
                const uint32_t last = b + DEPTH - 1U < blocks ? b + DEPTH - 1U : blocks;
                wait_stages_ahead<kQuadCopies>(last - 1U - b);
                if (b + DEPTH - 1U < blocks) source.start(slots[(s + DEPTH - 1) % DEPTH]);
                if (Q5K) quad_block_compute_q5k(slots[s], b, vd, vf, acc);
                else quad_block_compute(slots[s], b, vd, vf, acc);
            }
        }
    }
    float v = acc;
    v = v + xor1_f(v);          // acc0 + acc1 | acc2 + acc3
    v = v + xor2_f(v);          // (acc0 + acc1) + (acc2 + acc3)
    return v;
}

}  // namespace strix950
