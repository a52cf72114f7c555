// Q5_K x A8 gate / up rows: the second gate format of the reference's host executor
// (src/cpu/core/routed_expert.hpp:27 GateFormat::q5_k, arithmetic src/cpu/core/routed_expert.cpp:73-108 with Q5K). A block is
// 176 bytes: fp16 d, fp16 dmin, 12 factor bytes (as in Q4_K), 32 fifth-bit bytes (bit j of byte k belongs to element k of
// sub-block j), 128 nibble bytes; q = nibble | fifth bit << 4. Everything after the integer dot is the Q4_K pair term.
//
// sweep_q5k_row below reads its blocks straight from global memory; the projection kernel now streams the same blocks through
// the quad ring of q4k_quads.hpp (sweep_quads<DEPTH, true>: config 3 with Q5_K gate / up, 8 rows: 83.2 -> 78.4 us per layer) and
// this direct form stays as the plain statement of the arithmetic.
//
// Layout as in q4k_quads.hpp: 16 weight rows per wavefront, lane = (row, pair p); a lane owns the reference's pair
// accumulator p of its row and the row's value is (acc0 + acc1) + (acc2 + acc3) by two quad exchanges. A lane reads its
// part of a block straight from global memory: the header, the 32 fifth-bit bytes (shared by the quad) and the 32 nibble
// bytes of its pair.
#pragma once
#include "q4k_quads.hpp"

namespace strix950 {

constexpr uint32_t kQ5kBlock = 176;

// The value of one weight row against activation row `row` of `img`, for the lane's pair p; every lane of a quad returns it.
__device__ __forceinline__ float sweep_q5k_row(const uint8_t* wrow, uint32_t blocks, const A8Image& img, uint32_t row, uint32_t p) {
    const uint32_t groups = img.width / 32U;
    const u32x4* codes = reinterpret_cast<const u32x4*>(img.codes_of(row) + 64U * p);
    const float2* deltas = reinterpret_cast<const float2*>(img.deltas_of(row) + 2U * p);
    const int2* sums = reinterpret_cast<const int2*>(img.sums_of(row) + 2U * p);
    float acc = 0.0F;
#pragma unroll 4
    for (uint32_t b = 0; b < blocks; ++b) {     // four blocks of loads in flight: 52 -> 35 us at hidden 2048, 64 assignments
        const u32x4* blk = reinterpret_cast<const u32x4*>(wrow + static_cast<size_t>(b) * kQ5kBlock);
        const u32x4 hd = blk[0], h0 = blk[1], h1 = blk[2], q0 = blk[3U + 2U * p], q1 = blk[4U + 2U * p];
        const u32x4 c0 = codes[16U * b], c1 = codes[16U * b + 1U], c2 = codes[16U * b + 2U], c3 = codes[16U * b + 3U];
        const float2 e = deltas[4U * b];
        const int2 f = sums[4U * b];
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
        acc = acc + quad_pair_term(hd, p, dot0, dot1, e.x, e.y, static_cast<float>(f.x), static_cast<float>(f.y));
    }
    float v = acc;
    v = v + xor1_f(v);          // acc0 + acc1 | acc2 + acc3
    v = v + xor2_f(v);          // (acc0 + acc1) + (acc2 + acc3)
    return v;
}

}  // namespace strix950
