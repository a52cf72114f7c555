// Q6_K x A8 down rows (src/moe_a8_down_contract.cpp:18-37 q6k_a8_group_term, :147-158 evaluate_down_row type 14). A block
// is 210 bytes: 128 bytes of low nibbles, 64 bytes of high bit pairs, 16 signed scale bytes (one per 16 weights), fp16 d.
// Group j of a block (32 weights; half = j / 4, quarter = j % 4): weight i = (nibble | pair << 4) - 32 with
//   nibble = ql[64 half + 32 (quarter & 1) + i] >> (quarter >= 2 ? 4 : 0),  pair = qh[32 half + i] >> 2 quarter;
// integer = s[2j] * dot(first 16) + s[2j + 1] * dot(last 16) (exact), term = delta_g * (d * float(integer)); a block adds
// (term_2p + term_(2p+1)) to pair accumulator p, and the row's value is (acc0 + acc1) + (acc2 + acc3).
//
// Layout as in q4k_quads.hpp / down_groups.hpp: 16 output rows per wavefront, lane = (row, pair p), up to four assignments
// per weight pass. Both groups of a pair share `half`, so a lane reads 64 bytes of nibbles, 32 bytes of bit pairs and four
// scale bytes per block. Blocks are only 2-byte aligned (210 bytes): every multi-byte read is made of aligned words.
#pragma once
#include "device_math.hpp"
#include "q4k_rows.hpp"

namespace strix950 {

constexpr uint32_t kQ6kBlock = 210;

// N words starting at a 2-byte aligned address, from N + 1 aligned words
template <int N>
__device__ __forceinline__ void load_words_2aligned(const uint8_t* at, uint32_t (&out)[N]) {
    const uintptr_t address = reinterpret_cast<uintptr_t>(at);
    const uint32_t* aligned = reinterpret_cast<const uint32_t*>(address & ~static_cast<uintptr_t>(3));
    const uint32_t shift = static_cast<uint32_t>(address) & 3U;
    uint32_t raw[N + 1];
#pragma unroll
    for (int i = 0; i < N; ++i) raw[i] = aligned[i];
    raw[N] = shift ? aligned[N] : 0U;                         // an aligned start needs no straddling word: not read
#pragma unroll
    for (int i = 0; i < N; ++i) out[i] = __builtin_amdgcn_alignbyte(raw[i + 1], raw[i], shift);
}

__global__ __launch_bounds__(256) void down_q6k_kernel(mi355_moe_weights w, RowsK r, uint32_t assignments,
                                                       uint32_t items_at, uint32_t order_at) {
    typedef uint32_t u32x4_g __attribute__((ext_vector_type(4)));
    constexpr uint32_t NA = 4;
    const WorkItem item = work_item(w, r, items_at, blockIdx.y);
    const uint32_t e = item.e, begin = item.begin, end = item.end;
    if (begin == end) return;
    if (*r.job_status & MI355_STATUS_NONFINITE_PROJECTION) return;
    const uint32_t lane = threadIdx.x & 63U, wave = threadIdx.x >> 6, p = lane & 3U, half = p >> 1, odd = p & 1U;
    const uint32_t o = blockIdx.x * 64U + 16U * wave + (lane >> 2);
    const uint32_t groups = w.ffn / 32U, blocks = w.ffn / 256U;
    const uint8_t* wrow = w.down + static_cast<size_t>(e) * w.down_expert_stride + static_cast<size_t>(o) * w.down_row_stride;
    for (uint32_t c0 = begin; c0 < end; c0 += NA) {
        const uint32_t na = end - c0 < NA ? end - c0 : NA;
        uint32_t src[NA];
        float acc[NA];
        const int8_t* h_codes[NA];
        const float* h_deltas[NA];
#pragma unroll
        for (uint32_t a = 0; a < NA; ++a) {
            src[a] = ordered(r, order_at, c0 + (a < na ? a : na - 1U));
            acc[a] = 0.0F;
            h_codes[a] = r.h.codes_of(src[a]);
            h_deltas[a] = r.h.deltas_of(src[a]);
        }
#pragma unroll 2
        for (uint32_t b = 0; b < blocks; ++b) {
            const uint8_t* blk = wrow + static_cast<size_t>(b) * kQ6kBlock;
            uint32_t ql[16], qh[8];
            load_words_2aligned<16>(blk + 64U * half, ql);
            load_words_2aligned<8>(blk + 128U + 32U * half, qh);
            const uint16_t* tail = reinterpret_cast<const uint16_t*>(blk + 192U);
            const uint32_t sc01 = tail[2U * p], sc23 = tail[2U * p + 1U];          // scales 4p, 4p + 1 | 4p + 2, 4p + 3
            const float d = half_bits_to_float(tail[8]);
            // signed weights of groups 2p (k = 0) and 2p + 1 (k = 1), four per word
            uint32_t q[2][8];
#pragma unroll
            for (uint32_t k = 0; k < 2U; ++k)
#pragma unroll
                for (uint32_t i = 0; i < 8U; ++i) {
                    const uint32_t nibbles = (ql[8U * k + i] >> (4U * odd)) & 0x0f0f0f0fU;
                    const uint32_t pairs = (qh[i] >> (4U * odd + 2U * k)) & 0x03030303U;
                    const uint32_t six = nibbles | (pairs << 4);                   // 0 .. 63 per byte
                    q[k][i] = ((six | 0x80808080U) - 0x20202020U) ^ 0x80808080U;   // minus 32 per byte, no borrow between bytes
                }
            const int s[2][2] = {{static_cast<int8_t>(sc01 & 255U), static_cast<int8_t>(sc01 >> 8)},
                                 {static_cast<int8_t>(sc23 & 255U), static_cast<int8_t>(sc23 >> 8)}};
#pragma unroll
            for (uint32_t a = 0; a < NA; ++a) {
                if (a < na) {                                     // uniform over the workgroup
                    const u32x4_g* codes = reinterpret_cast<const u32x4_g*>(h_codes[a] + 256U * b + 64U * p);
                    const float2 delta = *reinterpret_cast<const float2*>(h_deltas[a] + 8U * b + 2U * p);
                    float term[2];
#pragma unroll
                    for (uint32_t k = 0; k < 2U; ++k) {
                        const u32x4_g c_lo = codes[2U * k], c_hi = codes[2U * k + 1U];
                        const uint32_t cw[8] = {c_lo.x, c_lo.y, c_lo.z, c_lo.w, c_hi.x, c_hi.y, c_hi.z, c_hi.w};
                        int first = 0, last = 0;
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            first = __builtin_amdgcn_sdot4(static_cast<int>(q[k][i]), static_cast<int>(cw[i]), first, false);
                            last = __builtin_amdgcn_sdot4(static_cast<int>(q[k][4 + i]), static_cast<int>(cw[4 + i]), last, false);
                        }
                        const int integer = s[k][0] * first + s[k][1] * last;
                        term[k] = (k == 0 ? delta.x : delta.y) * (d * static_cast<float>(integer));
                    }
                    acc[a] = acc[a] + (term[0] + term[1]);
                }
            }
        }
#pragma unroll
        for (uint32_t a = 0; a < NA; ++a) {
            if (a < na) {
                float v = acc[a];
                v = v + xor1_f(v);          // acc0 + acc1 | acc2 + acc3
                v = v + xor2_f(v);          // (acc0 + acc1) + (acc2 + acc3)
                if (p == 0) r.rawdots_of(src[a], w.hidden)[o] = v;
            }
        }
    }
}

}  // namespace strix950
