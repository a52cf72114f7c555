// Q4_K x A8 rows for a dense matrix (few long rows, 1..8 activation rows): one 64-lane wavefront evaluates 16 / AL weight
// rows, lane = (activation lane al, row r, pair p) with p in the low two bits. A lane owns the reference's pair
// accumulator p of its row (sub-blocks 2p and 2p + 1 of every super-block) for the activation rows al, al + AL, ...
//
// Why a second sweep: the row-per-lane sweep (q4k_rows.hpp) gives one wavefront per 64 rows, which is 80 wavefronts for a
// 5120-row matrix - far too few to pull HBM bandwidth, and K cannot be split without changing the summation order. The
// four pair accumulators of a row are independent chains, so this layout has 4 x (and with AL = 2, 8 x) as many
// wavefronts over the same rows, each streaming long contiguous pieces of its rows.
//
// A stage is 4 super-blocks (576 consecutive bytes) of each row plus, for every activation row, the 1,024 codes and the
// 32 group deltas / sums of the same 4 super-blocks; everything arrives by global_load_lds_dwordx4 through a ring of DEPTH
// slots (waits counted with s_waitcnt vmcnt). Weight piece c of row r sits at piece slot r * 36 + (c + r) % 36: the
// rotation keeps the lanes of different rows on different LDS banks.
//
// Arithmetic per (row, activation row): identical to q4k_rows.hpp; value = (acc0 + acc1) + (acc2 + acc3) by two DPP adds.
// Reference: src/cpu/core/routed_expert.cpp:73-108 == src/moe_q4k_a8_contract.cpp:126-140.
#pragma once
#include "q4k_rows.hpp"

namespace strix950 {

struct PairMatrix {
    const uint8_t* w;            // rows of Q4_K super-blocks
    uint64_t row_stride;         // bytes
    float* out;                  // out[a * out_stride + row]
    uint64_t out_stride;         // floats
};
struct PairArgs {
    PairMatrix m[2];             // blockIdx.y selects the matrix (gate / up share one launch)
    uint32_t rows;               // multiple of 16 / AL
    uint32_t blocks;             // super-blocks per row, multiple of 4
    A8Image img;                 // activation rows 0 .. nacts - 1 of this image
    uint32_t nacts;
    const uint32_t* skip_flag;   // optional: the launch does nothing when *skip_flag & skip_mask
    uint32_t skip_mask;
    RowsK publish;               // publish.top1_form != 0: matrix 0 holds a top-1 job's down rows, and each value's row output is published with it
};

constexpr uint32_t kPairBlocks = 4;                              // super-blocks per stage
// KL = 4 spreads the four super-blocks of a stage over four lanes as well (lane = (al, r, p, k), k in the low two bits):
// a quarter of the rows and of the instruction stream per wavefront, four times the wavefronts. The lanes of a quad then
// add their terms to the pair accumulator in super-block order (quad broadcasts), which keeps the reference's sum.
template <int AL, int KL = 1> constexpr uint32_t pair_rows() { return 16U / (AL * KL); }
template <int AL, int KL = 1> constexpr uint32_t pair_weight_copies() { return (pair_rows<AL, KL>() * 9U * kPairBlocks + 63U) / 64U; }
template <int NA, int AL, int KL = 1> constexpr uint32_t pair_copies() { return pair_weight_copies<AL, KL>() + NA * AL + 2U * ((NA * AL + 7U) / 8U); }
template <int NA, int AL, int KL = 1> constexpr uint32_t pair_slot_bytes() {
    return pair_weight_copies<AL, KL>() * 1024U + NA * AL * 1024U + 2U * ((NA * AL + 7U) / 8U) * 1024U;
}

template <int NA, int AL, int KL = 1>
struct PairSource {
    static constexpr uint32_t WC = pair_weight_copies<AL, KL>(), B = NA * AL, SC = (B + 7U) / 8U;
    const uint8_t* wp[WC];       // weight pieces
    const uint8_t* cp[B];        // activation codes: 16 bytes of row a per lane
    const uint8_t* dp[SC];       // deltas: lane l carries 16 bytes of row l / 8 (+ 8 per further copy)
    const uint8_t* sp[SC];
    __device__ __forceinline__ void init(const uint8_t* rows_base, uint32_t row_stride, const A8Image& img, uint32_t nacts) {
        const uint32_t lane = threadIdx.x & 63U, total = pair_rows<AL, KL>() * 36U;
#pragma unroll
        for (uint32_t i = 0; i < WC; ++i) {
            uint32_t j = i * 64U + lane;
            j = j < total ? j : total - 1U;                       // a short last copy repeats the last piece into unused LDS
            const uint32_t rr = __umulhi(j, 0x071C71C8U), t = j - 36U * rr;     // j / 36 exact for j < 576
            const uint32_t c = t >= rr ? t - rr : t + 36U - rr;
            wp[i] = rows_base + rr * row_stride + 16U * c;
        }
        const uint32_t groups = img.width / 32U;
#pragma unroll
        for (uint32_t a = 0; a < B; ++a) {
            const uint32_t row = a < nacts ? a : 0U;
            cp[a] = reinterpret_cast<const uint8_t*>(img.codes_of(row)) + 16U * lane;
        }
#pragma unroll
        for (uint32_t i = 0; i < SC; ++i) {
            const uint32_t a = 8U * i + (lane >> 3), row = a < nacts ? a : 0U;
            dp[i] = reinterpret_cast<const uint8_t*>(img.deltas_of(row)) + 16U * (lane & 7U);
            sp[i] = reinterpret_cast<const uint8_t*>(img.sums_of(row)) + 16U * (lane & 7U);
        }
    }
    // slot: [weights WC KiB][codes B KiB][deltas SC KiB][sums SC KiB]
    __device__ __forceinline__ void start(lds_u8* slot) {
#pragma unroll
        for (uint32_t i = 0; i < WC; ++i) {
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)wp[i],
                                             (__attribute__((address_space(3))) void*)(slot + 1024U * i), 16, 0, 0);
            wp[i] += kPairBlocks * 144U;
        }
#pragma unroll
        for (uint32_t a = 0; a < B; ++a) {
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)cp[a],
                                             (__attribute__((address_space(3))) void*)(slot + 1024U * (WC + a)), 16, 0, 0);
            cp[a] += kPairBlocks * 256U;
        }
#pragma unroll
        for (uint32_t i = 0; i < SC; ++i) {
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)dp[i],
                                             (__attribute__((address_space(3))) void*)(slot + 1024U * (WC + B + i)), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)sp[i],
                                             (__attribute__((address_space(3))) void*)(slot + 1024U * (WC + B + SC + i)), 16, 0, 0);
            dp[i] += kPairBlocks * 32U;
            sp[i] += kPairBlocks * 32U;
        }
    }
};

// The 4 super-blocks of one landed stage: the lane's (row r, pair p) against its NA activation rows.
template <int NA, int AL, int KL = 1>
__device__ __forceinline__ void pair_stage_compute(const lds_u8* slot, float (&acc)[NA]) {
    typedef const __attribute__((address_space(3))) u32x4 lds_u32x4;
    typedef const __attribute__((address_space(3))) float lds_f32;
    typedef const __attribute__((address_space(3))) int32_t lds_i32;
    constexpr uint32_t WC = pair_weight_copies<AL, KL>(), B = NA * AL, SC = (B + 7U) / 8U, RW = pair_rows<AL, KL>();
    const uint32_t lane = threadIdx.x & 63U, kl = KL == 4 ? lane & 3U : 0U, pl = KL == 4 ? lane >> 2 : lane;
    const uint32_t p = pl & 3U, r = (pl >> 2) & (RW - 1U), al = pl / (4U * RW);
    const lds_u8* wrow = slot + r * 576U;
    const lds_u8* codes = slot + 1024U * WC;
    const lds_u8* deltas = slot + 1024U * (WC + B);
    const lds_u8* sums = slot + 1024U * (WC + B + SC);
#pragma unroll
    for (uint32_t bb = 0; bb < kPairBlocks / KL; ++bb) {
        const uint32_t b = KL == 4 ? kl : bb;                  // KL = 4: the lane's own super-block of the stage
        // piece c of the row sits at slot (c + r) % 36
        uint32_t t0 = 9U * b + r, t1 = 9U * b + 1U + 2U * p + r, t2 = t1 + 1U;
        t0 = t0 >= 36U ? t0 - 36U : t0; t1 = t1 >= 36U ? t1 - 36U : t1; t2 = t2 >= 36U ? t2 - 36U : t2;
        const u32x4 hd = *(lds_u32x4*)(wrow + 16U * t0);
        const u32x4 q0 = *(lds_u32x4*)(wrow + 16U * t1), q1 = *(lds_u32x4*)(wrow + 16U * t2);
        const uint32_t w[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
        int lo[8], hi[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            lo[k] = static_cast<int>(w[k] & 0x0f0f0f0fU);
            hi[k] = static_cast<int>((w[k] >> 4) & 0x0f0f0f0fU);
        }
        // 6-bit scale / min of sub-blocks 2p, 2p + 1 (src/cpu/core/routed_expert.cpp:65-71)
        const uint32_t j0 = 2U * p, sh0 = 8U * (j0 & 3U), sh1 = sh0 + 8U;
        const uint32_t fa0 = (hd.y >> sh0) & 255U, fb0 = (hd.z >> sh0) & 255U, fc0 = (hd.w >> sh0) & 255U;
        const uint32_t fa1 = (hd.y >> sh1) & 255U, fb1 = (hd.z >> sh1) & 255U, fc1 = (hd.w >> sh1) & 255U;
        // branch-free choice between the two packings (pairs 0, 1: 6 low bits; pairs 2, 3: 4 + 2 split bits)
        const uint32_t lowmask = 0U - static_cast<uint32_t>(p < 2U);
        const auto pick = [lowmask](uint32_t lo6, uint32_t split) { return split ^ ((lo6 ^ split) & lowmask); };
        const uint32_t s0 = pick(fa0 & 63U, (fc0 & 15U) | ((fa0 >> 6) << 4)), m0 = pick(fb0 & 63U, (fc0 >> 4) | ((fb0 >> 6) << 4));
        const uint32_t s1 = pick(fa1 & 63U, (fc1 & 15U) | ((fa1 >> 6) << 4)), m1 = pick(fb1 & 63U, (fc1 >> 4) | ((fb1 >> 6) << 4));
        const float d = half_bits_to_float(hd.x & 0xffffU), dm = half_bits_to_float(hd.x >> 16);
        const float D0 = d * static_cast<float>(s0), M0 = dm * static_cast<float>(m0);
        const float D1 = d * static_cast<float>(s1), M1 = dm * static_cast<float>(m1);
#pragma unroll
        for (int i = 0; i < NA; ++i) {
            const uint32_t a = al + AL * i;
            lds_u32x4* c = (lds_u32x4*)(codes + 1024U * a + 256U * b + 64U * p);
            const u32x4 c0 = c[0], c1 = c[1], c2 = c[2], c3 = c[3];
            const uint32_t cw[16] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w, c2.x, c2.y, c2.z, c2.w, c3.x, c3.y, c3.z, c3.w};
            const uint32_t g = 128U * a + 32U * b + 8U * p;          // byte offset of the pair's two groups
            const float e0 = *(lds_f32*)(deltas + g), e1 = *(lds_f32*)(deltas + g + 4U);
            const float f0 = static_cast<float>(*(lds_i32*)(sums + g)), f1 = static_cast<float>(*(lds_i32*)(sums + g + 4U));
            int dot0 = 0, dot1 = 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                dot0 = __builtin_amdgcn_sdot4(lo[k], static_cast<int>(cw[k]), dot0, false);
                dot1 = __builtin_amdgcn_sdot4(hi[k], static_cast<int>(cw[8 + k]), dot1, false);
            }
            const float u0 = D0 * static_cast<float>(dot0), v0 = M0 * f0;
            const float u1 = D1 * static_cast<float>(dot1), v1 = M1 * f1;
            const float x0 = e0 * (u0 - v0), x1 = e1 * (u1 - v1);
            if constexpr (KL == 4) {
                // the quad's four terms, super-blocks 0..3 of the stage, in that order
                const int term = __builtin_bit_cast(int, x0 + x1);
                acc[i] = acc[i] + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(term, 0x00, 0xF, 0xF, true));
                acc[i] = acc[i] + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(term, 0x55, 0xF, 0xF, true));
                acc[i] = acc[i] + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(term, 0xAA, 0xF, 0xF, true));
                acc[i] = acc[i] + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(term, 0xFF, 0xF, 0xF, true));
            } else {
                acc[i] = acc[i] + (x0 + x1);
            }
            // many activation rows: keep the scheduler from hoisting every later row's operands at once (register pressure)
            if (NA > 2 && (i & 1) == 1) __builtin_amdgcn_sched_barrier(0);
        }
        if (NA > 2) __builtin_amdgcn_sched_barrier(0);
    }
}

template <int NA, int AL, int DEPTH, int KL = 1>
__global__ __launch_bounds__(64, 2) void q4k_pairs_kernel(PairArgs args) {
    __shared__ __attribute__((aligned(16))) uint8_t ring0[pair_slot_bytes<NA, AL, KL>()];
    __shared__ __attribute__((aligned(16))) uint8_t ring1[pair_slot_bytes<NA, AL, KL>()];
    __shared__ __attribute__((aligned(16))) uint8_t ring2[DEPTH > 2 ? pair_slot_bytes<NA, AL, KL>() : 16];
    __shared__ __attribute__((aligned(16))) uint8_t ring3[DEPTH > 3 ? pair_slot_bytes<NA, AL, KL>() : 16];
    lds_u8* const ring[4] = {(lds_u8*)ring0, (lds_u8*)ring1, (lds_u8*)ring2, (lds_u8*)ring3};
    if (args.skip_flag && (*args.skip_flag & args.skip_mask)) return;
    constexpr uint32_t RW = pair_rows<AL, KL>(), PER = pair_copies<NA, AL, KL>();
    const PairMatrix& m = args.m[blockIdx.y];
    const uint32_t row0 = blockIdx.x * RW, stages = args.blocks / kPairBlocks;
    PairSource<NA, AL, KL> source;
    source.init(m.w + static_cast<size_t>(row0) * m.row_stride, static_cast<uint32_t>(m.row_stride), args.img, args.nacts);
    float acc[NA];
#pragma unroll
    for (int i = 0; i < NA; ++i) acc[i] = 0.0F;
#pragma unroll
    for (int s = 0; s < DEPTH - 1; ++s)
        if (static_cast<uint32_t>(s) < stages) source.start(ring[s]);
    for (uint32_t b0 = 0; b0 < stages; b0 += DEPTH) {
#pragma unroll
        for (int s = 0; s < DEPTH; ++s) {
            const uint32_t b = b0 + s;
            if (b < stages) {
                const uint32_t last = b + DEPTH - 1U < stages ? b + DEPTH - 1U : stages;
                wait_stages_ahead<PER>(last - 1U - b);
                if (b + DEPTH - 1U < stages) source.start(ring[(s + DEPTH - 1) % DEPTH]);
                pair_stage_compute<NA, AL, KL>(ring[s], acc);
            }
        }
    }
    const uint32_t lane = threadIdx.x & 63U, kl = KL == 4 ? lane & 3U : 0U, pl = KL == 4 ? lane >> 2 : lane;
    const uint32_t p = pl & 3U, r = (pl >> 2) & (RW - 1U), al = pl / (4U * RW);
#pragma unroll
    for (int i = 0; i < NA; ++i) {
        float v = acc[i];
        if constexpr (KL == 4) {    // the pair index is lane bits 2, 3
            v = v + xor4_f(v);
            v = v + xor8_f(v);
        } else {
            v = v + xor1_f(v);      // acc0 + acc1 | acc2 + acc3
            v = v + xor2_f(v);      // (acc0 + acc1) + (acc2 + acc3)
        }
        const uint32_t a = al + AL * i;
        if (p == 0 && kl == 0 && a < args.nacts) {
            m.out[static_cast<size_t>(a) * m.out_stride + row0 + r] = v;
            if (args.publish.top1_form) args.publish.publish_top1(a, row0 + r, v);
        }
    }
}

}  // namespace strix950
