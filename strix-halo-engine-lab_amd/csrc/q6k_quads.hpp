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

// The same rows with the weights through LDS. Dense Q6_K rows lie back to back (210 * BLOCKS bytes each, 2-byte aligned), but
// the 16 rows of a wavefront together are one contiguous run of 3360 * BLOCKS bytes that starts on 16 bytes: the wave copies
// that run with aligned 16-byte global -> LDS pieces (no row structure, 1 KB per instruction) and the lanes then pick their
// 2-byte aligned words out of LDS with aligned 32-bit reads and a byte alignment, as the direct form does from global memory.
// The run of a wave for up to four super-blocks per row fits four workgroups' worth of LDS per compute unit; every copy of the
// launch is in flight before the first wave computes. Arithmetic and order are those of down_q6k_kernel.
template <int N>
__device__ __forceinline__ void lds_words_2aligned(const lds_u8* run, uint32_t at, uint32_t (&out)[N]) {
    typedef const __attribute__((address_space(3))) uint32_t lds_u32;
    lds_u32* aligned = reinterpret_cast<lds_u32*>(run + (at & ~3U));
    const uint32_t shift = at & 3U;
    uint32_t raw[N + 1];
#pragma unroll
    for (int i = 0; i <= N; ++i) raw[i] = aligned[i];           // (the word after an aligned run is inside the slot: read, unused)
#pragma unroll
    for (int i = 0; i < N; ++i) out[i] = __builtin_amdgcn_alignbyte(raw[i + 1], raw[i], shift);
}
template <int BLOCKS> constexpr uint32_t q6k_tile_copies() { return (210U * BLOCKS + 63U) / 64U; }      // 16 rows x 210 BLOCKS bytes in 16-byte pieces

template <int BLOCKS>
__global__ __launch_bounds__(256) void down_q6k_tile_kernel(mi355_moe_weights w, RowsK r, uint32_t assignments,
                                                            uint32_t items_at, uint32_t order_at) {
    typedef const __attribute__((address_space(3))) u32x4 lds_u32x4;
    typedef const __attribute__((address_space(3))) uint16_t lds_u16;
    typedef const __attribute__((address_space(3))) float lds_f32;
    constexpr uint32_t NA = 4, COPIES = q6k_tile_copies<BLOCKS>(), ROW = kQ6kBlock * BLOCKS, PIECES = 16U * ROW / 16U;
    constexpr uint32_t ACT = 1024U + 128U;                  // an activation row in LDS: its codes (256 BLOCKS bytes), at 1024 its group deltas
    __shared__ __attribute__((aligned(16))) uint8_t runs[4][COPIES * 1024U + 16U];
    __shared__ __attribute__((aligned(16))) uint8_t acts[NA][ACT];
    const WorkItem item = work_item(w, r, items_at, blockIdx.y);
    const uint32_t e = item.e, begin = item.begin, end = item.end;
    if (begin == end) return;                                                    // (uniform over the workgroup, like the next line)
    if (*r.job_status & MI355_STATUS_NONFINITE_PROJECTION) return;
    const uint32_t lane = threadIdx.x & 63U, wave = threadIdx.x >> 6, p = lane & 3U, half = p >> 1, odd = p & 1U;
    const uint32_t o = blockIdx.x * 64U + 16U * wave + (lane >> 2);
    lds_u8* const run = (lds_u8*)runs[wave];
    {
        // the wave's 16 rows: pieces 0 .. PIECES - 1 (a lane past the end repeats the last piece into the slot's padding)
        const uint8_t* chunk = w.down + static_cast<size_t>(e) * w.down_expert_stride + static_cast<size_t>(blockIdx.x * 64U + 16U * wave) * ROW;
#pragma unroll
        for (uint32_t c = 0; c < COPIES; ++c) {
            const uint32_t i = 64U * c + lane, piece = i < PIECES ? i : PIECES - 1U;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(chunk + 16U * piece),
                                             (__attribute__((address_space(3))) void*)(run + 1024U * c), 16, 0, 0);
        }
    }
    const uint32_t row_at = (lane >> 2) * ROW;
    for (uint32_t c0 = begin; c0 < end; c0 += NA) {
        const uint32_t na = end - c0 < NA ? end - c0 : NA;
        uint32_t src[NA];
        float acc[NA];
#pragma unroll
        for (uint32_t a = 0; a < NA; ++a) {
            src[a] = ordered(r, order_at, c0 + (a < na ? a : na - 1U));
            acc[a] = 0.0F;
        }
        // wave a brings activation row a of the pass: codes in pieces 0 .. 16 BLOCKS - 1, the group deltas behind them
        if (c0 != begin) __syncthreads();                                        // the rows of the last pass have been read
        if (wave < na) {
            const uint32_t mine = ordered(r, order_at, c0 + wave);
            lds_u8* const act = (lds_u8*)acts[wave];
            if (lane < 16U * BLOCKS)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(reinterpret_cast<const uint8_t*>(r.h.codes_of(mine)) + 16U * lane),
                                                 (__attribute__((address_space(3))) void*)act, 16, 0, 0);
            if (lane < 2U * BLOCKS)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(reinterpret_cast<const uint8_t*>(r.h.deltas_of(mine)) + 16U * lane),
                                                 (__attribute__((address_space(3))) void*)(act + 1024U), 16, 0, 0);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                         // the wave's weights (first pass) and its activation row
        __syncthreads();
#pragma unroll
        for (uint32_t b = 0; b < static_cast<uint32_t>(BLOCKS); ++b) {
            const uint32_t blk = row_at + b * kQ6kBlock;
            uint32_t ql[16], qh[8];
            lds_words_2aligned<16>(run, blk + 64U * half, ql);
            lds_words_2aligned<8>(run, blk + 128U + 32U * half, qh);
            lds_u16* tail = reinterpret_cast<lds_u16*>(run + blk + 192U);
            const uint32_t sc01 = tail[2U * p], sc23 = tail[2U * p + 1U];          // scales 4p, 4p + 1 | 4p + 2, 4p + 3
            const float d = half_bits_to_float(tail[8]);
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
                    lds_u32x4* codes = reinterpret_cast<lds_u32x4*>((lds_u8*)acts[a] + 256U * b + 64U * p);
                    lds_f32* delta = reinterpret_cast<lds_f32*>((lds_u8*)acts[a] + 1024U) + 8U * b + 2U * p;
                    float term[2];
#pragma unroll
                    for (uint32_t k = 0; k < 2U; ++k) {
                        const u32x4 c_lo = codes[2U * k], c_hi = codes[2U * k + 1U];
                        const uint32_t cw[8] = {c_lo.x, c_lo.y, c_lo.z, c_lo.w, c_hi.x, c_hi.y, c_hi.z, c_hi.w};
                        int first = 0, last = 0;
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            first = __builtin_amdgcn_sdot4(static_cast<int>(q[k][i]), static_cast<int>(cw[i]), first, false);
                            last = __builtin_amdgcn_sdot4(static_cast<int>(q[k][4 + i]), static_cast<int>(cw[4 + i]), last, false);
                        }
                        const int integer = s[k][0] * first + s[k][1] * last;
                        term[k] = delta[k] * (d * static_cast<float>(integer));
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

// Rows the LDS forms can copy: dense (back to back) from a 16-byte aligned start, and the A8 image of h in whole 16-byte
// pieces (the activation rows are copied to LDS as well).
inline bool q6k_tile_rows(const mi355_moe_weights& w, const RowsK& r) {
    return w.down_row_stride == static_cast<uint64_t>(kQ6kBlock) * (w.ffn / 256U) && reinterpret_cast<uintptr_t>(w.down) % 16U == 0 &&
           w.down_expert_stride % 16U == 0 && !r.h.table && reinterpret_cast<uintptr_t>(r.h.codes) % 16U == 0 &&
           reinterpret_cast<uintptr_t>(r.h.deltas) % 16U == 0 && r.h.codes_rs % 16U == 0 && r.h.deltas_rs % 16U == 0;
}

// Q6_K down rows of a launch: through LDS when the rows are dense (back to back) and at most four super-blocks long.
inline void launch_down_q6k(const mi355_moe_weights& w, const RowsK& r, dim3 grid, uint32_t assignments, uint32_t items_at, uint32_t order_at,
                            hipStream_t st) {
    const uint32_t blocks = w.ffn / 256U;
    const bool dense = q6k_tile_rows(w, r);
    if (dense && blocks == 1U) down_q6k_tile_kernel<1><<<grid, 256, 0, st>>>(w, r, assignments, items_at, order_at);
    else if (dense && blocks == 2U) down_q6k_tile_kernel<2><<<grid, 256, 0, st>>>(w, r, assignments, items_at, order_at);
    else if (dense && blocks == 3U) down_q6k_tile_kernel<3><<<grid, 256, 0, st>>>(w, r, assignments, items_at, order_at);
    else if (dense && blocks == 4U) down_q6k_tile_kernel<4><<<grid, 256, 0, st>>>(w, r, assignments, items_at, order_at);
    else down_q6k_kernel<<<grid, 256, 0, st>>>(w, r, assignments, items_at, order_at);
}

}  // namespace strix950
