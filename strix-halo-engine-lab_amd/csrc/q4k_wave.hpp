// Wave-level Q4_K x A8 row sweep for gfx950. One 64-lane wavefront (a one-wave workgroup) evaluates 64 weight rows
// (four row stages of 16 rows) against up to NB activation rows.
//
// HBM side: a stage is 16 weight rows x up to 4 super-blocks (576 consecutive bytes per row). The wave moves it straight
// from global memory into LDS with global_load_lds_dwordx4 (no VGPR round trip): each instruction's 64 lanes fetch 1 KiB
// of row-major 16-byte pieces, all 9 instructions of a stage are in flight together, so DRAM pages are consumed in
// bursts (a lane-per-row gather of the same bytes measured ~35 % lower bandwidth on MI355X). Two LDS buffers alternate:
// the copy of stage q + 1 is started before the arithmetic of stage q, and the buffers are separate __shared__ objects
// so that the compiler's wait-count tracking lets the reads of one buffer proceed while the other is being filled.
//
// LDS layout of a stage: piece c (16 bytes) of row r sits at piece slot r * P + ((c + r) mod P), P = 9 * super-blocks
// per row. The per-row rotation spreads the 16 rows over the LDS banks.
//
// Compute side: lane = 4 * rs + p. Row slot rs (0..15) is the lane's row of the stage; p (0..3) is the reference's
// pair index: the lane owns sub-blocks j = 2p (low nibbles) and 2p + 1 (high nibbles) of every super-block, i.e. the
// 32 quant bytes at block + 16 + 32 p. Per super-block b and activation row a:
//   x_j = E_g * ((D_j * float(dot_j)) - (DM_j * float(S_g))),  D_j = d * sc_j, DM_j = dmin * m_j, g = 8 b + j
//   acc[stage][a] += x_2p + x_2p+1          (b ascending: the lane's accumulator IS the reference's accum[p])
// and after the last super-block value = (acc_0 + acc_1) + (acc_2 + acc_3) by two DPP adds over the 4 lanes of a row.
// dot_j is one exact int32 sum of eight v_dot4_i32_i8.
// Reference arithmetic: src/cpu/core/routed_expert.cpp:73-108 == src/moe_q4k_a8_contract.cpp:126-140.
#pragma once
#include "device_math.hpp"

namespace strix950 {

__device__ uint32_t g_debug = 0;   // TEMP instrumentation

constexpr uint32_t kSegBlocks = 8;                          // super-blocks per activation segment (2048 elements)
constexpr uint32_t kHalfBlocks = 4;                         // super-blocks per weight stage
constexpr uint32_t kStageRows = 16;
constexpr uint32_t kStageBytes = kStageRows * kHalfBlocks * 144U;   // 9,216

template <int NB>
struct ActLds {                              // A8 images of up to NB activation rows, one K segment
    int8_t codes[NB][kSegBlocks * 256];
    float delta[NB][kSegBlocks * 8];
    float sumf[NB][kSegBlocks * 8];
};

struct A8Image {                             // device A8 image: codes [rows][width], deltas / sums [rows][width / 32]
    const int8_t* codes;
    const float* deltas;
    const int32_t* sums;
    uint32_t width;
};

// 6-bit scale / min of sub-block j from the three scale words of a header (src/cpu/core/routed_expert.cpp:65-71).
__device__ __forceinline__ void q4k_factors(const uint4& hd, uint32_t j, uint32_t& sc, uint32_t& mn) {
    const uint32_t shift = 8U * (j & 3U);
    const uint32_t fa = (hd.y >> shift) & 255U, fb = (hd.z >> shift) & 255U, fc = (hd.w >> shift) & 255U;
    sc = j < 4U ? (fa & 63U) : ((fc & 15U) | ((fa >> 6) << 4));
    mn = j < 4U ? (fb & 63U) : ((fc >> 4) | ((fb >> 6) << 4));
}

__device__ __forceinline__ int dot32(const int (&w)[8], const int4& c0, const int4& c1) {
    int d = 0;
    d = __builtin_amdgcn_sdot4(w[0], c0.x, d, false); d = __builtin_amdgcn_sdot4(w[1], c0.y, d, false);
    d = __builtin_amdgcn_sdot4(w[2], c0.z, d, false); d = __builtin_amdgcn_sdot4(w[3], c0.w, d, false);
    d = __builtin_amdgcn_sdot4(w[4], c1.x, d, false); d = __builtin_amdgcn_sdot4(w[5], c1.y, d, false);
    d = __builtin_amdgcn_sdot4(w[6], c1.z, d, false); d = __builtin_amdgcn_sdot4(w[7], c1.w, d, false);
    return d;
}

// Start the global -> LDS copy of one stage: rows base + r * row_stride (r < 16), bytes [blk0 * 144, (blk0 + nbs) * 144)
// of each row. Piece slot j of the stage is row r = j / P, slot t = j % P and receives piece (t - r) mod P of that row
// (no rotation for a one-super-block stage, P = 9 < 16). The division is a multiply-high by ceil(2^32 / P), exact here.
// Lanes past the end of a short stage re-fetch the last piece into the unused tail of the buffer.
__device__ __forceinline__ void stage_dma(uint8_t* lds_w, const uint8_t* base, uint32_t row_stride, uint32_t blk0, uint32_t nbs) {
    const uint32_t per_row = nbs * 9U, total = kStageRows * per_row, inv = 0xffffffffU / per_row + 1U;
    const uint8_t* src = base + static_cast<size_t>(blk0) * 144U;
    const uint32_t lane = threadIdx.x & 63U;
    const bool rotate = per_row >= kStageRows;
    for (uint32_t j0 = 0; j0 < total; j0 += 64U) {
        const uint32_t j = j0 + lane < total ? j0 + lane : total - 1U;
        const uint32_t r = __umulhi(j, inv), t = j - r * per_row;
        const uint32_t c = !rotate ? t : (t >= r ? t - r : t + per_row - r);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + r * row_stride + 16U * c),
                                         (__attribute__((address_space(3))) void*)(lds_w + 16U * j0), 16, 0, 0);
    }
}
// LDS byte offset of piece c of row r in a stage of per_row pieces per row.
__device__ __forceinline__ uint32_t stage_piece_at(uint32_t r, uint32_t c, uint32_t per_row, bool rotate) {
    uint32_t t = rotate ? c + r : c;
    t = t >= per_row ? t - per_row : t;
    return (r * per_row + t) * 16U;
}

// Arithmetic of one staged stage: the lane's row (rs) against na activation rows, nbs super-blocks.
// kb0 = index of the stage's first super-block inside the staged activation segment.
template <int NB>
__device__ __forceinline__ void stage_compute(const uint8_t* lds_w, const ActLds<NB>& lds, uint32_t kb0, uint32_t nbs, uint32_t na, float (&acc)[NB]) {
    const uint32_t lane = threadIdx.x & 63U, rs = lane >> 2, p = lane & 3U;
    const uint32_t per_row = nbs * 9U;
    const bool rotate = per_row >= kStageRows;
#pragma unroll 1
    for (uint32_t b = 0; b < nbs; ++b) {
        const uint4 hd = *reinterpret_cast<const uint4*>(lds_w + stage_piece_at(rs, 9U * b, per_row, rotate));
        const uint4 q0 = *reinterpret_cast<const uint4*>(lds_w + stage_piece_at(rs, 9U * b + 1U + 2U * p, per_row, rotate));
        const uint4 q1 = *reinterpret_cast<const uint4*>(lds_w + stage_piece_at(rs, 9U * b + 2U + 2U * p, per_row, rotate));
        const uint32_t q[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
        int lo[8], hi[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            lo[k] = static_cast<int>(q[k] & 0x0f0f0f0fU);
            hi[k] = static_cast<int>((q[k] >> 4) & 0x0f0f0f0fU);
        }
        uint32_t s0, m0, s1, m1;
        q4k_factors(hd, 2U * p, s0, m0);
        q4k_factors(hd, 2U * p + 1U, s1, m1);
        const float d = half_bits_to_float(hd.x & 0xffffU), dm = half_bits_to_float(hd.x >> 16);
        const float D0 = d * static_cast<float>(s0), M0 = dm * static_cast<float>(m0);
        const float D1 = d * static_cast<float>(s1), M1 = dm * static_cast<float>(m1);
        const uint32_t at = (kb0 + b) * 256U + 64U * p, g = (kb0 + b) * 8U + 2U * p;
#pragma unroll
        for (int a = 0; a < NB; ++a) {
            if (static_cast<uint32_t>(a) < na) {
                const int4* c = reinterpret_cast<const int4*>(&lds.codes[a][at]);
                const int4 c0 = c[0], c1 = c[1], c2 = c[2], c3 = c[3];
                const float2 e = *reinterpret_cast<const float2*>(&lds.delta[a][g]);
                const float2 s = *reinterpret_cast<const float2*>(&lds.sumf[a][g]);
                const int dot0 = dot32(lo, c0, c1), dot1 = dot32(hi, c2, c3);
                const float u0 = D0 * static_cast<float>(dot0), v0 = M0 * s.x;
                const float u1 = D1 * static_cast<float>(dot1), v1 = M1 * s.y;
                const float t0 = u0 - v0, t1 = u1 - v1;
                const float x0 = e.x * t0, x1 = e.y * t1;
                acc[a] = acc[a] + (x0 + x1);
            }
        }
    }
}

// Stage the A8 images of na activation rows for K elements [k0, k0 + kc).
template <int NB, class Index>
__device__ __forceinline__ void stage_images(ActLds<NB>& lds, const A8Image& img, Index src_row, uint32_t na, uint32_t k0, uint32_t kc) {
    const uint32_t lane = threadIdx.x & 63U, vec = kc / 16U;
    for (uint32_t i = lane; i < na * vec; i += 64U) {
        const uint32_t a = i / vec, c = i % vec;
        *reinterpret_cast<int4*>(&lds.codes[a][c * 16U]) =
            *reinterpret_cast<const int4*>(img.codes + static_cast<size_t>(src_row(a)) * img.width + k0 + c * 16U);
    }
    const uint32_t gc = kc / 32U, groups = img.width / 32U;
    for (uint32_t i = lane; i < na * gc; i += 64U) {
        const uint32_t a = i / gc, g = i % gc;
        const size_t at = static_cast<size_t>(src_row(a)) * groups + k0 / 32U + g;
        lds.delta[a][g] = img.deltas[at];
        lds.sumf[a][g] = static_cast<float>(img.sums[at]);
    }
}

// One activation segment (nbs <= 8 super-blocks starting at seg): row stages s = 0..3, each as one (HALVES = 1,
// nbs <= 4) or two (HALVES = 2) weight stages. Stage q uses LDS buffer q & 1; on entry stage 0's copy is under way, on
// exit the copy of the next segment's stage 0 (next_nbs super-blocks, 0 = none) is under way in buffer 0.
template <int NB, int HALVES>
__device__ __forceinline__ void sweep_segment(uint8_t* w0, uint8_t* w1, const ActLds<NB>& lds, const uint8_t* const (&stage_base)[4],
                                              uint32_t row_stride, uint32_t seg, uint32_t nbs, uint32_t next_nbs, uint32_t na,
                                              float (&acc)[4][NB]) {
    const uint32_t h0 = HALVES == 2 ? kHalfBlocks : nbs, h1 = nbs - h0;
#pragma unroll
    for (int q = 0; q < 4 * HALVES; ++q) {
        const int s = q / HALVES, half = q % HALVES;
        uint8_t* cur = (q & 1) ? w1 : w0;
        uint8_t* nxt = (q & 1) ? w0 : w1;
        __builtin_amdgcn_s_waitcnt(0);     // every outstanding copy (stage q) has landed
        __syncthreads();
        if (g_debug & 2) { if (!(g_debug & 1)) stage_compute<NB>(cur, lds, half ? h0 : 0U, half ? h1 : h0, na, acc[s]); continue; }
        if (q + 1 < 4 * HALVES) {
            const int ns = (q + 1) / HALVES, nh = (q + 1) % HALVES;
            stage_dma(nxt, stage_base[ns], row_stride, seg + (nh ? h0 : 0U), nh ? h1 : h0);
        } else if (next_nbs) {
            stage_dma(nxt, stage_base[0], row_stride, seg + kSegBlocks, next_nbs < kHalfBlocks ? next_nbs : kHalfBlocks);
        }
        if (!(g_debug & 1)) stage_compute<NB>(cur, lds, half ? h0 : 0U, half ? h1 : h0, na, acc[s]);
    }
}

// Whole sweep of a one-wave workgroup: 4 row stages of 16 rows (row stage s starts at stage_base[s], rows row_stride
// apart), K = blocks * 256 walked in activation segments of 8 super-blocks. acc[s][a] is the lane's pair accumulator of
// its row of row stage s. w0 / w1 are two separate LDS buffers of kStageBytes.
template <int NB, class Index>
__device__ __forceinline__ void sweep_rows(uint8_t* w0, uint8_t* w1, ActLds<NB>& lds, const uint8_t* const (&stage_base)[4], uint32_t row_stride,
                                           uint32_t blocks, const A8Image& img, Index src_row, uint32_t na, float (&acc)[4][NB]) {
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int a = 0; a < NB; ++a) acc[s][a] = 0.0F;
    __syncthreads();                           // earlier readers of the LDS buffers are done
    stage_dma(w0, stage_base[0], row_stride, 0, blocks < kHalfBlocks ? blocks : kHalfBlocks);
    for (uint32_t seg = 0; seg < blocks; seg += kSegBlocks) {
        const uint32_t left = blocks - seg, nbs = left < kSegBlocks ? left : kSegBlocks, next = left - nbs;
        if (seg) __syncthreads();              // the previous segment's arithmetic has finished reading the images
        stage_images<NB>(lds, img, src_row, na, seg * 256U, nbs * 256U);
        if (nbs > kHalfBlocks) sweep_segment<NB, 2>(w0, w1, lds, stage_base, row_stride, seg, nbs, next, na, acc);
        else sweep_segment<NB, 1>(w0, w1, lds, stage_base, row_stride, seg, nbs, next, na, acc);
    }
}

// (acc_0 + acc_1) + (acc_2 + acc_3) over the four lanes p of a row; every lane of the row receives the value.
__device__ __forceinline__ float row_tree4(float v) {
    v = v + xor1_f(v);
    v = v + xor2_f(v);
    return v;
}

// Reductions over the 16 row slots of a wave (lanes 4 rs + p, same p): strides 4, 8, 16, 32.
__device__ __forceinline__ float max_over_slots(float v) {
    v = __builtin_fmaxf(v, xor4_f(v)); v = __builtin_fmaxf(v, xor8_f(v)); v = __builtin_fmaxf(v, xor16_f(v));
    v = __builtin_fmaxf(v, __shfl_xor(v, 32));
    return v;
}
__device__ __forceinline__ int sum_over_slots(int v) {
    v += xor4_i(v); v += xor8_i(v); v += xor16_i(v);
    v += __shfl_xor(v, 32);
    return v;
}
__device__ __forceinline__ int or_over_slots(int v) {
    v |= xor4_i(v); v |= xor8_i(v); v |= xor16_i(v);
    v |= __shfl_xor(v, 32);
    return v;
}

}  // namespace strix950
