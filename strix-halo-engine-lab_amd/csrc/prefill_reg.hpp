// Prefill form of the routed experts for Q4_K tensors, second decomposition: every wave expands its own weight rows into
// MFMA operands in registers (no weight passes through LDS) and multiplies them with four 32-token tiles read from LDS.
// Same arithmetic class and exactness as prefill_f16.hpp (the reference's FAST forms, include/strix/cuda/qwen_moe.hpp:100-101;
// parity target: the exact-weight product, include/strix/ds41_layer.hpp:96-121): no weight is rounded.
//
// Arithmetic. w = d_b (sc_j q) - dmin_b m_j (src/ggml_dequant.cpp:119-130). The MFMA operand of a weight is the fp16 number
// 1024 + sc_j q, made by ONE integer multiply-add per two weights: (q1 << 16 | q0) * sc + 0x64006400 (sc q <= 945 < 1024
// stays inside the mantissa of 0x6400 = 1024.0). With S_bj[t] = sum of x_k[t] over sub-block j of super-block b,
//   out[t][f] = sum_b d_b[f] P_b[t][f] + sum_(b,j) S_bj[t] M_bj[f],
//   P_b = sum_(k in b) (1024 + sc_j q_k) x_k[t]  (fp16 MFMA, fp32 accumulation),   M_bj[f] = -(1024 d_b + dmin_b m_j).
// d_b is applied in fp32 once per super-block; the second sum is a K / 32-long product with S and M each carried as fp16
// hi + lo (three MFMAs per 16 sub-blocks). In the down product the activation h is carried as fp16 hi + lo as well (two
// MFMAs per operand pair), so that the only roundings of the whole expert are fp32 accumulations.
//
// Work decomposition. A plan item holds at most 128 rows of one expert. A 512-thread workgroup owns (item, 256 weight rows):
// 128 gate + 128 up rows (MODE 0) or 256 down rows (MODE 1). Wave w owns 32 of the rows x all 128 tokens: accumulators
// 4 token tiles x 16 registers for the super-block product P and the same for the running sum. K advances in stages of 64
// (one pair of sub-blocks = 32 quant bytes of a row): a lane (row n, half h) fetches the 16 quant bytes [16 h, 16 h + 16) of
// the pair straight into registers four stages ahead, expands them into the B operands of the stage's four MFMA k-steps
// (low nibbles: k-steps 0, 1; high nibbles: 2, 3), and the token rows of the stage (64 halves each) are copied global -> LDS
// three stages ahead through a 4-stage ring shared by the eight waves. One barrier per stage.
// MODE 0 pairs gate row f with up row f in lanes n and n + 16 of one wave, so SwiGLU needs one 16-lane exchange.
#pragma once
#include "prefill_f16.hpp"

namespace strix950 {

constexpr uint32_t kRgTokens = 128, kRgThreads = 512, kRgStageBytes = kRgTokens * 128U;   // one plane of one stage: 128 rows x 64 halves

// Number of vector-memory operations a wave issues in stage p (= stage % 4) of every super-block: the token copies of the
// stage three ahead, one quant fetch, and the header fetch (p = 0) or the sums copy (p = 1).
template <int MODE> __host__ __device__ constexpr uint32_t rg_token_ops() { return MODE == 1 ? 4U : 2U; }
template <int MODE> __host__ __device__ constexpr uint32_t rg_stage_ops(uint32_t p) { return rg_token_ops<MODE>() + 1U + (p < 2U ? 1U : 0U); }

// copy16_to_lds with the LDS address (lane 0's destination) already a scalar
__device__ __forceinline__ void copy16_to_lds_at(const uint8_t* src, uint32_t lds_at) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_at), "v"(src) : "memory", "m0");
}

template <int N> __device__ __forceinline__ void rg_wait() { asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory"); }

template <int MODE>
__global__ __launch_bounds__(kRgThreads) void prefill_reg_kernel(PrefillArgs a, uint32_t items_at, uint32_t order_at) {
    constexpr uint32_t PLANES = MODE == 1 ? 2U : 1U, NT = rg_token_ops<MODE>();
    __shared__ __attribute__((aligned(16))) uint8_t tok0[PLANES * kRgStageBytes];
    __shared__ __attribute__((aligned(16))) uint8_t tok1[PLANES * kRgStageBytes];
    __shared__ __attribute__((aligned(16))) uint8_t tok2[PLANES * kRgStageBytes];
    __shared__ __attribute__((aligned(16))) uint8_t tok3[PLANES * kRgStageBytes];
    __shared__ __attribute__((aligned(16))) uint8_t s_tile_mem[2][kRgTokens * 64U];        // [token][hi 16 | lo 16] sums of 16 sub-blocks
    __shared__ float part_sum[8][kRgTokens];                                               // MODE 0 epilogue: a wave's 16-feature sums of h
    pf_lds* const tok_stage[4] = {(pf_lds*)tok0, (pf_lds*)tok1, (pf_lds*)tok2, (pf_lds*)tok3};
    pf_lds* const s_tile = (pf_lds*)s_tile_mem;

    if (MODE == 1 && (*a.job_status & MI355_STATUS_NONFINITE_PROJECTION)) return;
    const uint32_t* order = a.plan + order_at;
    const uint32_t lane = threadIdx.x & 63U, wave = threadIdx.x >> 6, n31 = lane & 31U, half = lane >> 5;
    const uint32_t wave_s = __builtin_amdgcn_readfirstlane(wave);       // the wave's number as a scalar (LDS addresses of its copies)
    const uint32_t blocks = a.k / 256U, last_block = blocks - 1U, stages = a.k / 64U, last_stage = stages - 1U;
    const uint32_t last_group = (blocks + 1U) / 2U - 1U;
    const size_t sum_row = pf_sum_row_bytes(a.k);

    for (uint32_t unit = blockIdx.x; unit < a.units; unit += gridDim.x) {
    const uint32_t xcd = unit & 7U, q = unit >> 3;
    const uint32_t item_index = (q / a.tiles) * 8U + xcd, tile = q % a.tiles;
    if (item_index >= a.items) continue;
    const uint4 item = *reinterpret_cast<const uint4*>(a.plan + items_at + 4U * item_index);
    const uint32_t e = item.x, begin = item.y, count = item.z - item.y;
    if (count == 0) continue;

    // ---- the lane's weight row
    uint32_t feature;                                  // MODE 0: gate (n31 < 16) / up feature; MODE 1: output column
    const uint8_t* wbase = a.wa;
    if (MODE == 0) { feature = tile * 128U + 16U * wave + (n31 & 15U); if (n31 & 16U) wbase = a.wb; }
    else feature = tile * 256U + 32U * wave + n31;
    const uint8_t* wrow = wbase + static_cast<size_t>(e) * a.expert_stride + static_cast<size_t>(feature) * a.row_stride;

    // ---- token copies: copy i of a stage moves tile rows 8 (8 i + wave) .. + 8 of plane i / 2 (MODE 1); lane = (row % 8, slot)
    const uint8_t* tsrc[NT];
#pragma unroll
    for (uint32_t i = 0; i < NT; ++i) {
        const uint32_t row = 8U * (8U * (i & 1U) + wave) + (lane >> 3), tok = row < count ? row : count - 1U;
        const uint32_t piece = (lane & 7U) ^ ((row >> 1) & 7U);
        if (MODE == 0) tsrc[i] = a.x + static_cast<size_t>(order[begin + tok] / a.top_k) * a.x_stride + 16U * piece;
        // (h rows past the item's are other items' rows or the padding rows of the workspace: read, multiplied and never stored)
        else tsrc[i] = reinterpret_cast<const uint8_t*>((i < 2U ? a.h : a.h_lo) + static_cast<size_t>(begin + row) * a.k) + 16U * piece;
    }
    // ---- sums copy: piece = (token, part): parts 0, 1 = hi halves 0-7 / 8-15, parts 2, 3 = lo
    const uint8_t* ssrc;
    {
        const uint32_t row = threadIdx.x >> 2, part = threadIdx.x & 3U, tok = row < count ? row : count - 1U;
        const uint8_t* base = MODE == 0 ? a.x_sums + static_cast<size_t>(order[begin + tok] / a.top_k) * sum_row
                                        : a.h_sums + static_cast<size_t>(begin + tok) * sum_row;
        ssrc = base + 16U * (part & 1U) + (part >> 1) * (sum_row / 2U);
    }
    const auto copy_tokens = [&](uint32_t s, pf_lds* stage) {
        const uint32_t sc = s < last_stage ? s : last_stage;
        const uint32_t base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(stage)) + 1024U * wave_s;
#pragma unroll
        for (uint32_t i = 0; i < NT; ++i)
            copy16_to_lds_at(tsrc[i] + static_cast<size_t>(sc) * 128U, base + (i >> 1) * kRgStageBytes + 8192U * (i & 1U));
    };
    const auto copy_sums = [&](uint32_t g) {
        const uint32_t gc = g < last_group ? g : last_group;
        copy16_to_lds_at(ssrc + static_cast<size_t>(gc) * 32U,
                         static_cast<uint32_t>(reinterpret_cast<uintptr_t>(s_tile)) + (g & 1U) * (kRgTokens * 64U) + 1024U * wave_s);
    };
    const auto fetch_header = [&](uint32_t b, u32x4& hd) {
        const uint8_t* blk = wrow + static_cast<size_t>(b < last_block ? b : last_block) * 144U;
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(hd) : "v"(blk) : "memory");
    };
    const auto fetch_quants = [&](uint32_t s, u32x4& qs) {
        const uint32_t sc = s < last_stage ? s : last_stage;
        const uint8_t* at = wrow + static_cast<size_t>(sc >> 2) * 144U + 16U + 32U * (sc & 3U) + 16U * half;
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(qs) : "v"(at) : "memory");
    };

    // ---- expansion: 8 nibbles (low or high) of two quant words -> the B operand of one k-step: four registers of two fp16
    // numbers 1024 + sc q each
    uint32_t magic;
    asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(magic));
    const auto expand = [&](uint32_t w0, uint32_t w1, uint32_t sc) -> half8 {
        const uint32_t r0 = __builtin_amdgcn_perm(0U, w0, 0x0c010c00U), r1 = __builtin_amdgcn_perm(0U, w0, 0x0c030c02U);
        const uint32_t r2 = __builtin_amdgcn_perm(0U, w1, 0x0c010c00U), r3 = __builtin_amdgcn_perm(0U, w1, 0x0c030c02U);
        const u32x4 v = {r0 * sc + magic, r1 * sc + magic, r2 * sc + magic, r3 * sc + magic};
        return __builtin_bit_cast(half8, v);
    };
    // sc of sub-blocks 2 p and 2 p + 1 (src/cpu/core/routed_expert.cpp:65-71)
    const auto scales = [&](const u32x4& hd, uint32_t p, uint32_t& s_lo, uint32_t& s_hi) {
        const uint32_t sh0 = 16U * (p & 1U), sh1 = sh0 + 8U;
        const uint32_t fa0 = (hd.y >> sh0) & 255U, fc0 = (hd.w >> sh0) & 255U, fa1 = (hd.y >> sh1) & 255U, fc1 = (hd.w >> sh1) & 255U;
        s_lo = p < 2U ? (fa0 & 63U) : ((fc0 & 15U) | ((fa0 >> 6) << 4));
        s_hi = p < 2U ? (fa1 & 63U) : ((fc1 & 15U) | ((fa1 >> 6) << 4));
    };

    // Everything from the first fetch to the last store is instantiated per number of token tiles that hold a row of the item
    // (the other tiles are neither read nor multiplied). The weight fetches are plain instructions the compiler does not
    // track, so a register they write must stay reserved until the fetch has landed - including the (clamped) fetches of a
    // unit's last stages that nothing uses: they are awaited at the end of the instantiation, and no fetched register is
    // live across a join of two instantiations (a join may copy registers, and a copy of a register whose fetch is still in
    // flight would copy stale data).
    const auto run_unit = [&](auto live_constant) __attribute__((always_inline)) {
    constexpr uint32_t LIVE = decltype(live_constant)::value;
    floatx16 acc[4], part[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) { acc[i][j] = 0.0F; part[i][j] = 0.0F; }
    const uint32_t trow = n31 * 128U, sw = (n31 >> 1) & 7U;
    uint32_t piece_at[4];                              // k-step j reads piece (j >= 2 ? 4 : 0) + 2 half + (j & 1) of the lane's token row
#pragma unroll
    for (uint32_t j = 0; j < 4U; ++j) piece_at[j] = ((((j >> 1) << 2) + 2U * half + (j & 1U)) ^ sw) << 4;

    // ---- prologue: the operations of "stages -3, -2, -1" in the loop's own order, so that its counts hold from the first
    // stage on; before them the header and the quants of stage 0
    u32x4 hd_cur, hd_next = {0U, 0U, 0U, 0U}, qs[4];
    u32x4 mreg_hi = {0U, 0U, 0U, 0U}, mreg_lo = {0U, 0U, 0U, 0U};      // B operand of the S x M product: -(1024 d + dmin m_j), j = 8 half .. + 8
    fetch_header(0, hd_cur); fetch_quants(0, qs[0]);
    copy_tokens(0, tok_stage[0]); copy_sums(0); fetch_quants(1, qs[1]);
    copy_tokens(1, tok_stage[1]); fetch_quants(2, qs[2]);
    copy_tokens(2, tok_stage[2]); fetch_quants(3, qs[3]);
    // younger than the token copies of stage 0: sums + quants, then two stages of NT + 1
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(hd_cur), "+v"(qs[0]) : "n"(2U * NT + 4U) : "memory");
    pf_barrier();

    half8 bfrag;                                       // B operand of the next k-step
    {
        uint32_t s_lo, s_hi;
        scales(hd_cur, 0, s_lo, s_hi);
        bfrag = expand(qs[0].x & 0x0f0f0f0fU, qs[0].y & 0x0f0f0f0fU, s_lo);
    }

    {
        const auto stage = [&](auto p_constant, uint32_t b) __attribute__((always_inline)) {
                constexpr uint32_t p = decltype(p_constant)::value;
                const uint32_t s = 4U * b + p;
                // ---- issue: token copies three stages ahead, the header of the next super-block / the sums of the next group
                copy_tokens(s + 3U, tok_stage[(p + 3U) & 3U]);
                if (p == 0) fetch_header(b + 1U, hd_next);
                if (p == 1) copy_sums((b >> 1) + 1U);
                uint32_t s_lo, s_hi;
                scales(hd_cur, p, s_lo, s_hi);
                const u32x4 qw = qs[p];
                const pf_lds* tok = tok_stage[p] + trow;
                // The stage's MFMAs as a flat sequence of slots m = (k-step j, plane, token tile i); the A operand of slot m + W is
                // requested right after the MFMA of slot m into the registers that MFMA has just read (a window of W operands).
                constexpr uint32_t PER = PLANES * LIVE, N = 4U * PER, W = N < 4U ? N : 4U;
                half8 frag[W];
                const auto request = [&](uint32_t m) __attribute__((always_inline)) {
                    const uint32_t j = m / PER, pl = (m / LIVE) % PLANES, i = m % LIVE;
                    frag[m % W] = *reinterpret_cast<const __attribute__((address_space(3))) half8*>(tok + pl * kRgStageBytes + i * 32U * 128U + piece_at[j]);
                };
#pragma unroll
                for (uint32_t m = 0; m < W; ++m) request(m);
                half8 bcur = bfrag;
#pragma unroll
                for (uint32_t m = 0; m < N; ++m) {
                    const uint32_t j = m / PER, i = m % LIVE;
                    if (m % PER == 0) {
                        // a new k-step: take its B operand and expand the next one while this k-step multiplies
                        bcur = bfrag;
                        if (j == 0) bfrag = expand(qw.z & 0x0f0f0f0fU, qw.w & 0x0f0f0f0fU, s_lo);
                        else if (j == 1) bfrag = expand((qw.x >> 4) & 0x0f0f0f0fU, (qw.y >> 4) & 0x0f0f0f0fU, s_hi);
                        else if (j == 2) {
                            bfrag = expand((qw.z >> 4) & 0x0f0f0f0fU, (qw.w >> 4) & 0x0f0f0f0fU, s_hi);
                            fetch_quants(s + 4U, qs[p]);             // the stage's quant registers are free now
                        } else {
                            // first k-step of the next stage: its quants were fetched at the end of stage s - 3 (younger operations:
                            // the whole of stages s - 2, s - 1 and s), its header - when it opens a super-block - in stage s - 3
                            constexpr uint32_t pn = (p + 1U) & 3U;
                            constexpr uint32_t younger = rg_stage_ops<MODE>((p + 2U) & 3U) + rg_stage_ops<MODE>((p + 3U) & 3U) + rg_stage_ops<MODE>(p);
                            if (p == 3U) asm volatile("s_waitcnt vmcnt(%2)" : "+v"(qs[pn]), "+v"(hd_next) : "n"(younger) : "memory");
                            else asm volatile("s_waitcnt vmcnt(%1)" : "+v"(qs[pn]) : "n"(younger) : "memory");
                            uint32_t n_lo, n_hi;
                            scales(p == 3U ? hd_next : hd_cur, pn, n_lo, n_hi);
                            bfrag = expand(qs[pn].x & 0x0f0f0f0fU, qs[pn].y & 0x0f0f0f0fU, n_lo);
                        }
                    }
                    if (p == 0 && m < LIVE) {                        // first MFMA of a super-block's product: it starts from zero
                        const floatx16 zero = {0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F};
                        part[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(frag[m % W], bcur, zero, 0, 0, 0);
                    } else {
                        part[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(frag[m % W], bcur, part[i], 0, 0, 0);
                    }
                    if (m + W < N) request(m + W);
                    // the scheduler otherwise sinks the request down to its use (registers are scarce) and the MFMA then waits
                    // for the whole LDS round trip: nothing moves across this point (1874 -> 1828 us gate / up, 1642 -> 1565 us down)
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (p == 1U) {
                    // this lane's M operand: the eight sub-blocks of super-block 2 g + half of the group
                    if ((b & 1U) == half) {
                        const float d = half_bits_to_float(hd_cur.x & 0xffffU), dm = half_bits_to_float(hd_cur.x >> 16);
                        const float d1024 = 1024.0F * d;
                        uint32_t mh[4], ml[4];
#pragma unroll
                        for (int jj = 0; jj < 8; jj += 2) {
                            float v[2];
#pragma unroll
                            for (int t = 0; t < 2; ++t) {
                                const uint32_t sh = 8U * ((jj + t) & 3U);
                                const uint32_t mn = (jj + t) < 4 ? ((hd_cur.z >> sh) & 63U) : (((hd_cur.w >> (sh + 4U)) & 15U) | (((hd_cur.z >> (sh + 6U)) & 3U) << 4));
                                v[t] = -(d1024 + dm * static_cast<float>(mn));
                            }
                            const half2v hh = __builtin_convertvector(float2v{v[0], v[1]}, half2v);
                            mh[jj / 2] = __builtin_bit_cast(uint32_t, hh);
                            ml[jj / 2] = pack_half2(v[0] - static_cast<float>(hh.x), v[1] - static_cast<float>(hh.y));
                        }
                        mreg_hi = u32x4{mh[0], mh[1], mh[2], mh[3]};
                        mreg_lo = u32x4{ml[0], ml[1], ml[2], ml[3]};
                    } else if ((b & 1U) == 0 && b + 1U == blocks) {  // odd count: the last group's second super-block does not exist
                        mreg_hi = u32x4{0U, 0U, 0U, 0U};
                        mreg_lo = u32x4{0U, 0U, 0U, 0U};
                    }
                }
                if (p == 3U) {
                    // end of a super-block: running sum += d * P
                    const float d = half_bits_to_float(hd_cur.x & 0xffffU);
#pragma unroll
                    for (uint32_t i = 0; i < LIVE; ++i)
#pragma unroll
                        for (int r = 0; r < 16; ++r) acc[i][r] = __builtin_fmaf(d, part[i][r], acc[i][r]);
                    if ((b & 1U) || b + 1U == blocks) {
                        // end of a group of 16 sub-blocks: running sum += S hi * M hi + S lo * M hi + S hi * M lo
                        const pf_lds* st = s_tile + ((b >> 1) & 1U) * (kRgTokens * 64U) + n31 * 64U + 16U * half;
                        const half8 mh = __builtin_bit_cast(half8, mreg_hi), ml = __builtin_bit_cast(half8, mreg_lo);
#pragma unroll
                        for (uint32_t i = 0; i < LIVE; ++i) {
                            const half8 sh = *reinterpret_cast<const __attribute__((address_space(3))) half8*>(st + i * 32U * 64U);
                            const half8 sl = *reinterpret_cast<const __attribute__((address_space(3))) half8*>(st + i * 32U * 64U + 32U);
                            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(sh, mh, acc[i], 0, 0, 0);
                            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(sl, mh, acc[i], 0, 0, 0);
                            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(sh, ml, acc[i], 0, 0, 0);
                        }
                    }
                    hd_cur = hd_next;
                }
                // the token copies of stage s + 1 were issued at the start of stage s - 2: younger operations = the rest of that
                // stage and the whole of stages s - 1 and s
                constexpr uint32_t younger_tokens = rg_stage_ops<MODE>((p + 2U) & 3U) - NT + rg_stage_ops<MODE>((p + 3U) & 3U) + rg_stage_ops<MODE>(p);
                rg_wait<static_cast<int>(younger_tokens)>();
                pf_barrier();
        };
        for (uint32_t b = 0; b < blocks; ++b) {
            stage(std::integral_constant<uint32_t, 0>{}, b);
            stage(std::integral_constant<uint32_t, 1>{}, b);
            stage(std::integral_constant<uint32_t, 2>{}, b);
            stage(std::integral_constant<uint32_t, 3>{}, b);
        }
    }

    // ---- epilogue. Result layout of a 32 x 32 tile: the lane holds weight row n31; register r is token 8 (r / 4) + 4 half + r % 4
    if (MODE == 0) {
        // Lane n31 < 16 holds gate row f of 16 tokens per tile, lane n31 + 16 the up row of the same feature. The two lanes
        // swap halves (the gate lane sends its tokens 8-15, the up lane its tokens 0-7), so each evaluates SwiGLU for eight
        // tokens. This class follows the exact product to a tolerance, so exp and the division are the hardware's
        // (v_exp_f32, v_rcp_f32: one ulp each).
        const uint32_t f_out = tile * 128U + 16U * wave + (n31 & 15U);
        const bool gate_lane = n31 < 16U;
#pragma unroll
        for (uint32_t i = 0; i < LIVE; ++i)
#pragma unroll
            for (uint32_t k = 0; k < 8U; ++k) {
                // (the two registers are named before the per-lane choice: choosing the INDEX per lane instead would make the
                // compiler walk all sixteen registers of the tile with compare-and-select pairs)
                float first = acc[i][k], second = acc[i][8U + k];
                asm volatile("" : "+v"(first), "+v"(second));
                const float sent = gate_lane ? second : first, got = xor16_f(sent);
                const float g = gate_lane ? first : got, u = gate_lane ? got : second;
                const uint32_t r = gate_lane ? k : 8U + k;
                const uint32_t t = 32U * i + 8U * (r / 4U) + 4U * half + (r & 3U);
                const bool live = t < count;
                float gc = g, uc = u;
                swiglu_clamp(gc, uc, a.swiglu_limit);
                const float hv = (gc * __builtin_amdgcn_rcpf(1.0F + __builtin_amdgcn_exp2f(gc * -1.44269504F))) * uc;
                const _Float16 h_hi = static_cast<_Float16>(hv);
                const _Float16 h_lo = static_cast<_Float16>(hv - static_cast<float>(h_hi));
                float sum = live ? static_cast<float>(h_hi) + static_cast<float>(h_lo) : 0.0F;
                sum += xor1_f(sum); sum += xor2_f(sum); sum += xor4_f(sum); sum += xor8_f(sum);     // over the wave's 16 features
                if ((n31 & 15U) == 0) part_sum[wave][t] = sum;    // a sub-block of 32 features is two waves' halves
                if (live) {
                    const size_t at = static_cast<size_t>(begin + t) * a.features + f_out;
                    a.h[at] = h_hi;
                    a.h_lo[at] = h_lo;
                    if (!(finite_f(g) && finite_f(u) && finite_f(static_cast<float>(h_hi)))) {     // h beyond fp16 counts as non-finite
                        atomicOr(pf_status_of(a, order[begin + t]), static_cast<uint32_t>(MI355_STATUS_NONFINITE_PROJECTION));
                        atomicOr(a.job_status, static_cast<uint32_t>(MI355_STATUS_NONFINITE_PROJECTION));
                    }
                }
            }
        __syncthreads();
        if (threadIdx.x < 4U * kRgTokens) {
            const uint32_t t = threadIdx.x & (kRgTokens - 1U), pair = threadIdx.x / kRgTokens;      // sub-block tile * 4 + pair of this tile
            if (t < count) {
                const float sum = part_sum[2U * pair][t] + part_sum[2U * pair + 1U][t];
                _Float16* sums = reinterpret_cast<_Float16*>(a.h_sums + static_cast<size_t>(begin + t) * pf_sum_row_bytes(a.features));
                split_half(sum, sums[tile * 4U + pair], sums[pf_sum_slots(a.features) + tile * 4U + pair]);
            }
        }
        __syncthreads();                                  // part_sum is free for the next unit
    } else {
        const uint32_t f_out = tile * 256U + 32U * wave + n31;
#pragma unroll
        for (uint32_t i = 0; i < LIVE; ++i)
#pragma unroll
            for (uint32_t r = 0; r < 16U; ++r) {
                const uint32_t t = 32U * i + 8U * (r / 4U) + 4U * half + (r & 3U);
                if (t < count) pf_rawdots_of(a, order[begin + t])[f_out] = a.rawdots_bf16 ? pf_round_bf16(acc[i][r]) : acc[i][r];
            }
    }
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(hd_cur), "+v"(hd_next), "+v"(qs[0]), "+v"(qs[1]), "+v"(qs[2]), "+v"(qs[3]) : : "memory");
    };
    const uint32_t live_tiles = (count + 31U) / 32U;
    if (live_tiles >= 4U) run_unit(std::integral_constant<uint32_t, 4>{});
    else if (live_tiles == 3U) run_unit(std::integral_constant<uint32_t, 3>{});
    else if (live_tiles == 2U) run_unit(std::integral_constant<uint32_t, 2>{});
    else run_unit(std::integral_constant<uint32_t, 1>{});
    }   // units
}

}  // namespace strix950
