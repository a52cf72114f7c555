// Q4_K x A8 rows with one super-block per lane: the sweep whose stages are contiguous runs of memory.
//
// Rows in dense GGUF order lie back to back: R rows of B super-blocks are R * B * 144 consecutive bytes. A stage is such a
// run - R * B <= 64 blocks, R the largest power of two that fits - copied global -> LDS as whole 1 KB pieces (a read-only
// stream of this shape was measured at 20.6 us for 113 MB in 1536 waves against 22.6 us when a stage is one 144-byte block of
// each of 64 rows 1152 bytes apart; 11.8 against 14.4 us for the 57 MB of 2048 waves x 3 stages). Lane l of the first R * B
// evaluates block l % B of row l / B of the stage: the lane's block index never changes, so its share of the activation row
// - 256 codes, 8 deltas, 8 sums - is loaded once into registers and no activation operand goes through LDS. A row's value is
// the reference's chain over its blocks in ascending order,
//   acc[p] = (((0 + t_0[p]) + t_1[p]) + ...) + t_(B-1)[p],  t_b[p] = x_2p + x_2p+1 of block b,  value = (acc0 + acc1) + (acc2 + acc3),
// run across the row's B neighbouring lanes as B - 1 shift-and-add steps (a whole-wave DPP shift by one lane), so the bits are
// those of q4k_rows.hpp's lane-per-row sweep. One activation row per sweep.
// Reference arithmetic: src/cpu/core/routed_expert.cpp:73-108 == src/moe_q4k_a8_contract.cpp:126-140.
#pragma once
#include "q4k_rows.hpp"

namespace strix950 {

struct BlockLanes { uint32_t B, R, used, stage_bytes; };
constexpr uint32_t kBlockLaneCopies = 9;        // copy instructions per stage (a stage is at most 9,216 bytes)
// max_rows: the rows of one contiguous run (a power of two)
__host__ __device__ inline bool block_lanes_ok(uint32_t B, uint32_t max_rows) { return B >= 1U && B <= 64U && max_rows >= 1U; }
__host__ __device__ inline BlockLanes block_lanes(uint32_t B, uint32_t max_rows) {
    uint32_t R = 1;
    while (2U * R * B <= 64U && 2U * R <= max_rows) R *= 2U;
    return BlockLanes{B, R, R * B, R * B * 144U};
}

// At most N copies outstanding, and every LDS read of this wave returned. The second half matters: a copy writes LDS when its
// data arrives, not in the order of the wave's LDS instructions - a read of a slot that is still queued in the LDS when the next
// copy into that slot lands returns the new bytes (seen with eight waves per workgroup reading 29 KB each while a stage that hit in
// the caches came back in under a microsecond). So a slot is overwritten only after the reads of it have returned.
template <int N> __device__ __forceinline__ void block_lane_wait() { __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (0 << 8)); }

__device__ __forceinline__ float wave_shr1(float v) {       // lane l receives lane l - 1's value (lane 0: 0)
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x138, 0xF, 0xF, true));
}

// stage_base(s): first byte of stage s (16-byte aligned). Returns, in lane i < stages * R, the value of row i (rows in stage
// order) against image row `image_row` of img; other lanes: 0. slots: DEPTH separate LDS objects of >= 9,216 bytes with
// nothing in flight; on exit every copy has landed and been consumed.
template <int DEPTH, class StageBase>
__device__ __forceinline__ float sweep_block_lanes(lds_u8* const (&slots)[DEPTH], StageBase stage_base, uint32_t stages, const BlockLanes g,
                                                   const A8Image& img, uint32_t image_row) {
    typedef const __attribute__((address_space(3))) u32x4 lds_u32x4;
    const uint32_t lane = threadIdx.x & 63U;
    const bool active = lane < g.used;
    const uint32_t b = active ? lane % g.B : 0U, r_in_stage = lane / g.B;
    // every copy instruction moves 64 pieces of 16 bytes; the pieces past the stage's end re-read its first piece into the slot's
    // unused tail, so that each stage is the same number of operations and the waits can count them
    uint32_t piece_offset[kBlockLaneCopies];
#pragma unroll
    for (uint32_t i = 0; i < kBlockLaneCopies; ++i) {
        const uint32_t at = (i * 64U + lane) * 16U;
        piece_offset[i] = at < g.stage_bytes ? at : 0U;
    }
    const auto start = [&](uint32_t s, lds_u8* slot) {
        const uint8_t* base = stage_base(s);
#pragma unroll
        for (uint32_t i = 0; i < kBlockLaneCopies; ++i)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(base + piece_offset[i]),
                                             (__attribute__((address_space(3))) void*)(slot + 1024U * i), 16, 0, 0);
    };
#pragma unroll
    for (int s = 0; s < DEPTH - 1; ++s)
        if (static_cast<uint32_t>(s) < stages) start(static_cast<uint32_t>(s), slots[s]);
    // the lane's share of the activation row: block b's 256 codes, 8 deltas, 8 sums
    u32x4 code[16];
    float delta[8], fsum[8];
    {
        const u32x4* cs = reinterpret_cast<const u32x4*>(img.codes_of(image_row) + 256U * b);
#pragma unroll
        for (int i = 0; i < 16; ++i) code[i] = cs[i];
        const f32x4* ds = reinterpret_cast<const f32x4*>(img.deltas_of(image_row) + 8U * b);
        const f32x4 d0 = ds[0], d1 = ds[1];
        typedef int i32x4 __attribute__((ext_vector_type(4)));
        const i32x4* ss = reinterpret_cast<const i32x4*>(img.sums_of(image_row) + 8U * b);
        const i32x4 s0 = ss[0], s1 = ss[1];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            delta[j] = d0[j]; delta[4 + j] = d1[j];
            fsum[j] = static_cast<float>(s0[j]); fsum[4 + j] = static_cast<float>(s1[j]);
        }
    }
    float value = 0.0F;
    for (uint32_t s0 = 0; s0 < stages; s0 += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const uint32_t s = s0 + d;
            if (s < stages) {
                // started so far: stages 0 .. min(stages, s + DEPTH - 1) - 1; stage s must have landed (the activation loads, issued
                // after the first DEPTH - 1 stages, are older than every later stage)
                const uint32_t last = s + DEPTH - 1U < stages ? s + DEPTH - 1U : stages, ahead = last - 1U - s;
                if (ahead == 0) block_lane_wait<0>();
                else if (ahead == 1) block_lane_wait<kBlockLaneCopies>();
                else if (ahead == 2) block_lane_wait<2 * kBlockLaneCopies>();
                else block_lane_wait<3 * kBlockLaneCopies>();
                if (s + DEPTH - 1U < stages) start(s + DEPTH - 1U, slots[(d + DEPTH - 1) % DEPTH]);
                lds_u32x4* blk = (lds_u32x4*)(slots[d] + (active ? lane : 0U) * 144U);
                const u32x4 hd = blk[0];
                u32x4 q[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) q[i] = blk[1 + i];
                const float dd = half_bits_to_float(hd.x & 0xffffU), dm = half_bits_to_float(hd.x >> 16);
                uint32_t sc[8], mn[8];
                q4k_factors<0>(hd, sc[0], mn[0]); q4k_factors<1>(hd, sc[1], mn[1]); q4k_factors<2>(hd, sc[2], mn[2]); q4k_factors<3>(hd, sc[3], mn[3]);
                q4k_factors<4>(hd, sc[4], mn[4]); q4k_factors<5>(hd, sc[5], mn[5]); q4k_factors<6>(hd, sc[6], mn[6]); q4k_factors<7>(hd, sc[7], mn[7]);
                float t[4];
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    const uint32_t wq[8] = {q[2 * p].x, q[2 * p].y, q[2 * p].z, q[2 * p].w, q[2 * p + 1].x, q[2 * p + 1].y, q[2 * p + 1].z, q[2 * p + 1].w};
                    const uint32_t c[16] = {code[4 * p].x, code[4 * p].y, code[4 * p].z, code[4 * p].w, code[4 * p + 1].x, code[4 * p + 1].y, code[4 * p + 1].z, code[4 * p + 1].w,
                                            code[4 * p + 2].x, code[4 * p + 2].y, code[4 * p + 2].z, code[4 * p + 2].w, code[4 * p + 3].x, code[4 * p + 3].y, code[4 * p + 3].z, code[4 * p + 3].w};
                    int dot0 = 0, dot1 = 0;
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        dot0 = __builtin_amdgcn_sdot4(static_cast<int>(wq[k] & 0x0f0f0f0fU), static_cast<int>(c[k]), dot0, false);
                        dot1 = __builtin_amdgcn_sdot4(static_cast<int>((wq[k] >> 4) & 0x0f0f0f0fU), static_cast<int>(c[8 + k]), dot1, false);
                    }
                    const float D0 = dd * static_cast<float>(sc[2 * p]), D1 = dd * static_cast<float>(sc[2 * p + 1]);
                    const float M0 = dm * static_cast<float>(mn[2 * p]), M1 = dm * static_cast<float>(mn[2 * p + 1]);
                    const float u0 = D0 * static_cast<float>(dot0), v0 = M0 * fsum[2 * p];
                    const float u1 = D1 * static_cast<float>(dot1), v1 = M1 * fsum[2 * p + 1];
                    const float t0 = u0 - v0, t1 = u1 - v1;
                    const float x0 = delta[2 * p] * t0, x1 = delta[2 * p + 1] * t1;
                    t[p] = x0 + x1;
                }
                // the row's chain over its blocks: after step i the lanes of blocks 0..i hold their prefix
                float acc[4];
#pragma unroll
                for (int p = 0; p < 4; ++p) acc[p] = 0.0F + t[p];
                for (uint32_t step = 1; step < g.B; ++step) {
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        const float chained = wave_shr1(acc[p]) + t[p];
                        acc[p] = b == 0 ? acc[p] : chained;
                    }
                }
                const float row_value = (acc[0] + acc[1]) + (acc[2] + acc[3]);      // valid in the lane of the row's last block
                // row i of the stage sits in lane i * B + B - 1; the sweep's row s * R + i belongs in lane s * R + i
                for (uint32_t i = 0; i < g.R; ++i) {
                    const int got = __builtin_amdgcn_readlane(__builtin_bit_cast(int, row_value), static_cast<int>(i * g.B + g.B - 1U));
                    value = lane == s * g.R + i ? __builtin_bit_cast(float, got) : value;
                }
                (void)r_in_stage;
            }
        }
    }
    return value;
}

// The same sweep for stages that fill the wave (R * B = 64) and a stage count known at compile time, with the rows' chains taken
// out of the stages: every stage leaves its block's four pair terms in registers; after the last stage the terms are laid out in
// LDS in block order (stage s, lane l at 16 (64 s + l) bytes of slot 0, which nothing copies into any more) and lane i = sweep row
// i = stage i / R, row i % R of it, adds the B terms of its row in ascending order - the additions of the shift-and-add chain,
// in its order, once per sweep instead of B - 1 whole-wave steps and R lane broadcasts per stage (at B = 8: 43 vector
// instructions and 16 LDS accesses per sweep in the place of 114 per stage). STAGES * 1 KB must fit a slot.
template <int STAGES, class StageBase>
__device__ __forceinline__ float sweep_block_lanes_terms(lds_u8* const (&slots)[2], StageBase stage_base, const BlockLanes g, const A8Image& img, uint32_t image_row) {
    static_assert(STAGES >= 2 && STAGES <= 9, "terms of every stage side by side in one slot");
    typedef const __attribute__((address_space(3))) u32x4 lds_u32x4;
    typedef const __attribute__((address_space(3))) f32x4 lds_f32x4;
    typedef __attribute__((address_space(3))) f32x4 lds_f32x4_w;
    const uint32_t lane = threadIdx.x & 63U;
    const uint32_t b = lane % g.B;
    const auto start = [&](uint32_t s, lds_u8* slot) {
        const uint8_t* base = stage_base(s) + 16U * lane;
#pragma unroll
        for (uint32_t i = 0; i < kBlockLaneCopies; ++i)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(base + 1024U * i),
                                             (__attribute__((address_space(3))) void*)(slot + 1024U * i), 16, 0, 0);
    };
    start(0U, slots[0]);
    // the lane's share of the activation row: block b's 256 codes, 8 deltas, 8 sums
    u32x4 code[16];
    float delta[8], fsum[8];
    {
        const u32x4* cs = reinterpret_cast<const u32x4*>(img.codes_of(image_row) + 256U * b);
#pragma unroll
        for (int i = 0; i < 16; ++i) code[i] = cs[i];
        const f32x4* ds = reinterpret_cast<const f32x4*>(img.deltas_of(image_row) + 8U * b);
        const f32x4 d0 = ds[0], d1 = ds[1];
        typedef int i32x4 __attribute__((ext_vector_type(4)));
        const i32x4* ss = reinterpret_cast<const i32x4*>(img.sums_of(image_row) + 8U * b);
        const i32x4 s0 = ss[0], s1 = ss[1];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            delta[j] = d0[j]; delta[4 + j] = d1[j];
            fsum[j] = static_cast<float>(s0[j]); fsum[4 + j] = static_cast<float>(s1[j]);
        }
    }
    float t[STAGES][4];
#pragma unroll
    for (int S = 0; S < STAGES; ++S) {
        // stage S has landed (the activation loads are older than every stage after the first), the reads of the slot the next copy
        // goes into have returned
        block_lane_wait<0>();
        if (S + 1 < STAGES) start(static_cast<uint32_t>(S + 1), slots[(S + 1) % 2]);
        lds_u32x4* blk = (lds_u32x4*)(slots[S % 2] + lane * 144U);
        const u32x4 hd = blk[0];
        u32x4 q[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) q[i] = blk[1 + i];
        const float dd = half_bits_to_float(hd.x & 0xffffU), dm = half_bits_to_float(hd.x >> 16);
        uint32_t sc[8], mn[8];
        q4k_factors<0>(hd, sc[0], mn[0]); q4k_factors<1>(hd, sc[1], mn[1]); q4k_factors<2>(hd, sc[2], mn[2]); q4k_factors<3>(hd, sc[3], mn[3]);
        q4k_factors<4>(hd, sc[4], mn[4]); q4k_factors<5>(hd, sc[5], mn[5]); q4k_factors<6>(hd, sc[6], mn[6]); q4k_factors<7>(hd, sc[7], mn[7]);
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const uint32_t wq[8] = {q[2 * p].x, q[2 * p].y, q[2 * p].z, q[2 * p].w, q[2 * p + 1].x, q[2 * p + 1].y, q[2 * p + 1].z, q[2 * p + 1].w};
            const uint32_t c[16] = {code[4 * p].x, code[4 * p].y, code[4 * p].z, code[4 * p].w, code[4 * p + 1].x, code[4 * p + 1].y, code[4 * p + 1].z, code[4 * p + 1].w,
                                    code[4 * p + 2].x, code[4 * p + 2].y, code[4 * p + 2].z, code[4 * p + 2].w, code[4 * p + 3].x, code[4 * p + 3].y, code[4 * p + 3].z, code[4 * p + 3].w};
            int dot0 = 0, dot1 = 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                dot0 = __builtin_amdgcn_sdot4(static_cast<int>(wq[k] & 0x0f0f0f0fU), static_cast<int>(c[k]), dot0, false);
                dot1 = __builtin_amdgcn_sdot4(static_cast<int>((wq[k] >> 4) & 0x0f0f0f0fU), static_cast<int>(c[8 + k]), dot1, false);
            }
            const float D0 = dd * static_cast<float>(sc[2 * p]), D1 = dd * static_cast<float>(sc[2 * p + 1]);
            const float M0 = dm * static_cast<float>(mn[2 * p]), M1 = dm * static_cast<float>(mn[2 * p + 1]);
            const float u0 = D0 * static_cast<float>(dot0), v0 = M0 * fsum[2 * p];
            const float u1 = D1 * static_cast<float>(dot1), v1 = M1 * fsum[2 * p + 1];
            const float t0 = u0 - v0, t1 = u1 - v1;
            const float x0 = delta[2 * p] * t0, x1 = delta[2 * p + 1] * t1;
            t[S][p] = x0 + x1;
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");            // the last stage's reads have returned: slot 0 is free for the terms
#pragma unroll
    for (int S = 0; S < STAGES; ++S) *((lds_f32x4_w*)(slots[0] + 16U * (64U * static_cast<uint32_t>(S) + lane))) = f32x4{t[S][0], t[S][1], t[S][2], t[S][3]};
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    // sweep row `lane`: stage lane / R, blocks (lane % R) * B .. + B - 1 of it
    const uint32_t first = 64U * (lane / g.R) + (lane % g.R) * g.B;
    float acc[4] = {0.0F, 0.0F, 0.0F, 0.0F};
    for (uint32_t k = 0; k < g.B; ++k) {
        const f32x4 term = *((lds_f32x4*)(slots[0] + 16U * (first + k)));
#pragma unroll
        for (int p = 0; p < 4; ++p) acc[p] = acc[p] + term[p];
    }
    const float value = (acc[0] + acc[1]) + (acc[2] + acc[3]);
    return lane < static_cast<uint32_t>(STAGES) * g.R ? value : 0.0F;
}

// ---------------------------------------------------------------------------------------------------------------- flat rows
// 64 dense rows of B super-blocks against ONE activation row, as the byte stream they are: 64 * B blocks = B stages of 64 blocks,
// each stage 9,216 contiguous bytes (nine 1 KB pieces). Lane l of stage s evaluates block g = 64 s + l, which is block g % B of
// row g / B, so the lane's activation share changes from stage to stage: the row's A8 image (codes, deltas, sums: 320 B bytes)
// is copied to LDS once and every lane reads its block's 320 bytes from there. The four pair terms of every block are kept in
// registers; at the end they are laid out in LDS in block order, where lane r finds the terms of its row's B blocks side by
// side and adds them in ascending order: acc[p] = ((0 + t_0[p]) + t_1[p]) + ..., value = (acc0 + acc1) + (acc2 + acc3) - the
// reference's chain (src/cpu/core/routed_expert.cpp:73-108), the bits of the lane-per-row sweep.
// slots: DEPTH separate LDS objects of >= 9,216 bytes (slot 0 also serves the final exchange: B * 1 KB), act: >= 320 * B bytes of LDS;
// nothing in flight on entry, everything landed and consumed on exit.
constexpr uint32_t kFlatStageBytes = 9216;
__host__ __device__ constexpr uint32_t flat_act_bytes(uint32_t B) { return 320U * B; }

template <int B, int DEPTH>
__device__ __forceinline__ float sweep_flat_rows(lds_u8* const (&slots)[DEPTH], lds_u8* act, const uint8_t* rows, const A8Image& img, uint32_t image_row) {
    static_assert(B >= 1 && B <= 9 && DEPTH >= 2 && DEPTH <= 4, "flat rows: 1..9 super-blocks per row (the exchange fits slot 0), ring of 2..4 slots");
    typedef const __attribute__((address_space(3))) u32x4 lds_u32x4;
    typedef const __attribute__((address_space(3))) f32x4 lds_f32x4;
    typedef int i32x4 __attribute__((ext_vector_type(4)));
    typedef const __attribute__((address_space(3))) i32x4 lds_i32x4;
    const uint32_t lane = threadIdx.x & 63U;
    const auto start = [&](uint32_t s, lds_u8* slot) {
        const uint8_t* base = rows + static_cast<size_t>(s) * kFlatStageBytes + 16U * lane;
#pragma unroll
        for (uint32_t i = 0; i < kBlockLaneCopies; ++i)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(base + 1024U * i),
                                             (__attribute__((address_space(3))) void*)(slot + 1024U * i), 16, 0, 0);
    };
#pragma unroll
    for (int s = 0; s < DEPTH - 1; ++s)
        if (s < B) start(static_cast<uint32_t>(s), slots[s]);
    // (behind the first stage, not in front of it: the stage's address waits for the work item, the image's for nothing - issued
    // first, the image's copy would be waited for together with the work item and the stage would start a round trip late)
    // the activation row: codes 256 B | deltas 32 B | sums 32 B bytes, in pieces of 16 (20 B pieces, at most three copy instructions)
    constexpr uint32_t kActPieces = 20U * B, kActCopies = (kActPieces + 63U) / 64U;
    {
        const uint8_t* codes = reinterpret_cast<const uint8_t*>(img.codes_of(image_row));
        const uint8_t* deltas = reinterpret_cast<const uint8_t*>(img.deltas_of(image_row));
        const uint8_t* sums = reinterpret_cast<const uint8_t*>(img.sums_of(image_row));
#pragma unroll
        for (uint32_t i = 0; i < kActCopies; ++i) {
            const uint32_t piece = i * 64U + lane;
            const uint8_t* src = piece < 16U * B ? codes + 16U * piece : piece < 18U * B ? deltas + 16U * (piece - 16U * B) : sums + 16U * (piece - 18U * B);
            if (piece < kActPieces)                                // (the lanes past the image copy nothing)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src, (__attribute__((address_space(3))) void*)(act + 1024U * i), 16, 0, 0);
        }
    }
    float t[B][4];
#pragma unroll
    for (int s = 0; s < B; ++s) {
        // started so far: the activation image and stages 0 .. min(B, s + DEPTH - 1) - 1; stage s (and everything older) must have landed
        const int last = s + DEPTH - 1 < B ? s + DEPTH - 1 : B, ahead = last - 1 - s;
        asm volatile("" ::: "memory");          // a stage's LDS reads stay inside the stage (hoisted, the three activation shares alone fill the register file)
        if (ahead == 0 || s == 0) block_lane_wait<0>();      // (stage 0 also waits for the image, the youngest copy so far)
        else if (ahead == 1) block_lane_wait<kBlockLaneCopies>();
        else if (ahead == 2) block_lane_wait<2 * kBlockLaneCopies>();
        else block_lane_wait<3 * kBlockLaneCopies>();
        if (s + DEPTH - 1 < B) start(static_cast<uint32_t>(s + DEPTH - 1), slots[(s + DEPTH - 1) % DEPTH]);
        const uint32_t b = (64U * static_cast<uint32_t>(s) + lane) % static_cast<uint32_t>(B);
        u32x4 code[16];
        float delta[8], fsum[8];
        lds_u32x4* cs = (lds_u32x4*)(act + 256U * b);
#pragma unroll
        for (int i = 0; i < 16; ++i) code[i] = cs[i];
        lds_f32x4* ds = (lds_f32x4*)(act + 256U * B + 32U * b);
        const f32x4 d0 = ds[0], d1 = ds[1];
        lds_i32x4* ss = (lds_i32x4*)(act + 288U * B + 32U * b);
        const i32x4 s0 = ss[0], s1 = ss[1];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            delta[j] = d0[j]; delta[4 + j] = d1[j];
            fsum[j] = static_cast<float>(s0[j]); fsum[4 + j] = static_cast<float>(s1[j]);
        }
        lds_u32x4* blk = (lds_u32x4*)(slots[s % DEPTH] + lane * 144U);
        const u32x4 hd = blk[0];
        u32x4 q[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) q[i] = blk[1 + i];
        const float dd = half_bits_to_float(hd.x & 0xffffU), dm = half_bits_to_float(hd.x >> 16);
        uint32_t sc[8], mn[8];
        q4k_factors<0>(hd, sc[0], mn[0]); q4k_factors<1>(hd, sc[1], mn[1]); q4k_factors<2>(hd, sc[2], mn[2]); q4k_factors<3>(hd, sc[3], mn[3]);
        q4k_factors<4>(hd, sc[4], mn[4]); q4k_factors<5>(hd, sc[5], mn[5]); q4k_factors<6>(hd, sc[6], mn[6]); q4k_factors<7>(hd, sc[7], mn[7]);
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const uint32_t wq[8] = {q[2 * p].x, q[2 * p].y, q[2 * p].z, q[2 * p].w, q[2 * p + 1].x, q[2 * p + 1].y, q[2 * p + 1].z, q[2 * p + 1].w};
            const uint32_t c[16] = {code[4 * p].x, code[4 * p].y, code[4 * p].z, code[4 * p].w, code[4 * p + 1].x, code[4 * p + 1].y, code[4 * p + 1].z, code[4 * p + 1].w,
                                    code[4 * p + 2].x, code[4 * p + 2].y, code[4 * p + 2].z, code[4 * p + 2].w, code[4 * p + 3].x, code[4 * p + 3].y, code[4 * p + 3].z, code[4 * p + 3].w};
            int dot0 = 0, dot1 = 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                dot0 = __builtin_amdgcn_sdot4(static_cast<int>(wq[k] & 0x0f0f0f0fU), static_cast<int>(c[k]), dot0, false);
                dot1 = __builtin_amdgcn_sdot4(static_cast<int>((wq[k] >> 4) & 0x0f0f0f0fU), static_cast<int>(c[8 + k]), dot1, false);
            }
            const float D0 = dd * static_cast<float>(sc[2 * p]), D1 = dd * static_cast<float>(sc[2 * p + 1]);
            const float M0 = dm * static_cast<float>(mn[2 * p]), M1 = dm * static_cast<float>(mn[2 * p + 1]);
            const float u0 = D0 * static_cast<float>(dot0), v0 = M0 * fsum[2 * p];
            const float u1 = D1 * static_cast<float>(dot1), v1 = M1 * fsum[2 * p + 1];
            const float t0 = u0 - v0, t1 = u1 - v1;
            const float x0 = delta[2 * p] * t0, x1 = delta[2 * p + 1] * t1;
            t[s][p] = x0 + x1;
        }
    }
    // the terms in block order: block g at 16 g bytes of slot 0 (every read of the slots has returned: the terms depend on them)
    typedef __attribute__((address_space(3))) f32x4 lds_f32x4_w;
#pragma unroll
    for (int s = 0; s < B; ++s) *((lds_f32x4_w*)(slots[0] + 16U * (64U * static_cast<uint32_t>(s) + lane))) = f32x4{t[s][0], t[s][1], t[s][2], t[s][3]};
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");            // one wave: its own stores are visible to its own later reads once issued in order
    float acc[4] = {0.0F, 0.0F, 0.0F, 0.0F};
#pragma unroll
    for (int b = 0; b < B; ++b) {
        const f32x4 term = *((lds_f32x4*)(slots[0] + 16U * (static_cast<uint32_t>(B) * lane + static_cast<uint32_t>(b))));
#pragma unroll
        for (int p = 0; p < 4; ++p) acc[p] = acc[p] + term[p];
    }
    return (acc[0] + acc[1]) + (acc[2] + acc[3]);
}

}  // namespace strix950
