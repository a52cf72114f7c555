// Wave-level Q4_K x A8 row sweep for gfx950. One 64-lane wavefront (a one-wave workgroup) evaluates 64 weight rows,
// lane = row, against NA activation rows that are common to the whole wave.
//
// HBM side: a stage is one super-block (144 bytes) of each of the 64 rows = 9,216 bytes = 576 16-byte pieces. The wave
// moves it straight from global memory into LDS with nine global_load_lds_dwordx4 (no VGPR round trip); piece j of the
// stage is piece j % 9 of row j / 9 and lands at LDS byte 16 j, so a row's block is 144 consecutive LDS bytes. DEPTH LDS
// buffers form a ring: the copies of stages b + 1 .. b + DEPTH - 1 are in flight while stage b is evaluated. The ring
// slots are separate __shared__ objects so that the compiler's wait-count tracking lets the reads of one slot proceed
// while the others are being filled.
//
// LDS side: lane r reads its nine pieces with ds_read_b128 at r * 144 + 16 c; the 36-word row pitch makes every group
// of eight lanes cover all banks, so the reads are conflict free without padding.
//
// Activation side: the A8 image (codes, deltas, sums) of an activation row is the same for every lane, so it is read
// through the constant address space with wave-uniform addresses: the compiler emits scalar loads, and the codes feed
// v_dot4_i32_i8 as scalar operands. No activation byte passes through LDS or a VGPR.
//
// Arithmetic per row, super-block b ascending, pair p = 0..3 (sub-blocks j = 2p: low nibbles, 2p + 1: high nibbles):
//   x_j = E_g * ((D_j * float(dot_j)) - (DM_j * float(S_g))),  D_j = d * sc_j, DM_j = dmin * m_j, g = 8 b + j
//   acc[a][p] += x_2p + x_2p+1
// and after the last super-block value = (acc_0 + acc_1) + (acc_2 + acc_3), all inside the lane. dot_j is one exact
// int32 sum of eight v_dot4_i32_i8.
// Reference arithmetic: src/cpu/core/routed_expert.cpp:73-108 == src/moe_q4k_a8_contract.cpp:126-140.
#pragma once
#include "device_math.hpp"

namespace strix950 {

constexpr uint32_t kWaveRows = 64;
constexpr uint32_t kStageBytes = kWaveRows * 144U;   // 9,216
constexpr uint32_t kStagePieces = 9;                 // global_load_lds instructions per stage (576 pieces / 64 lanes)

typedef uint32_t u32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
#define STRIX_CONSTANT __attribute__((address_space(4)))

struct A8Image {                             // device A8 image: codes [rows][width], deltas / sums [rows][width / 32]
    const int8_t* codes;
    const float* deltas;
    const int32_t* sums;
    uint32_t width;
};

// Per-lane source pointers of the nine pieces the lane copies in every stage. row_ptr(r) = first byte of row r (0..63).
struct StageSource {
    const uint8_t* piece[kStagePieces];
    template <class RowPtr>
    __device__ __forceinline__ void init(RowPtr row_ptr) {
        const uint32_t lane = threadIdx.x & 63U;
#pragma unroll
        for (uint32_t i = 0; i < kStagePieces; ++i) {
            const uint32_t j = i * 64U + lane, r = __umulhi(j, 0x1C71C71DU), c = j - 9U * r;   // j / 9 exact for j < 576
            piece[i] = row_ptr(r) + 16U * c;
        }
    }
    // start the copy of the next super-block of all 64 rows into one ring slot, then step to the block after it
    __device__ __forceinline__ void start(uint8_t* slot) {
#pragma unroll
        for (uint32_t i = 0; i < kStagePieces; ++i) {
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)piece[i],
                                             (__attribute__((address_space(3))) void*)(slot + 1024U * i), 16, 0, 0);
            piece[i] += 144;
        }
    }
};

// s_waitcnt vmcnt(N): at most N vector memory operations (here: stage copies, nine per stage) still outstanding.
template <int N>
__device__ __forceinline__ void wait_copies() {
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}
__device__ __forceinline__ void wait_stages_ahead(uint32_t ahead) {   // ahead = stages started after the one needed
    if (ahead == 0) wait_copies<0>();
    else if (ahead == 1) wait_copies<9>();
    else if (ahead == 2) wait_copies<18>();
    else wait_copies<27>();
}

// 6-bit scale / min of sub-block J (compile-time) from the three scale words of a block header
// (src/cpu/core/routed_expert.cpp:65-71).
template <int J>
__device__ __forceinline__ void q4k_factors(const u32x4& hd, uint32_t& sc, uint32_t& mn) {
    constexpr uint32_t shift = 8U * (J & 3);
    if (J < 4) {
        sc = (hd.y >> shift) & 63U;
        mn = (hd.z >> shift) & 63U;
    } else {
        sc = ((hd.w >> shift) & 15U) | (((hd.y >> (shift + 6U)) & 3U) << 4);
        mn = ((hd.w >> (shift + 4U)) & 15U) | (((hd.z >> (shift + 6U)) & 3U) << 4);
    }
}

// Uniform view of the NA activation rows of one sweep. The codes are read with scalar loads of 64 bytes (one pair's
// 64 codes); the group deltas and sums are held one group per lane (64 groups = 8 super-blocks per refill) and
// broadcast with v_readlane.
template <int NA>
struct ActRows {
    const STRIX_CONSTANT u32x16* codes[NA];    // row base, wave-uniform
    const float* deltas[NA];                   // row base
    const int32_t* sums[NA];
    uint32_t groups;                           // per activation row
    __device__ __forceinline__ ActRows(const A8Image& img, const uint32_t (&row)[NA]) : groups(img.width / 32U) {
#pragma unroll
        for (int a = 0; a < NA; ++a) {
            const uint32_t r = __builtin_amdgcn_readfirstlane(row[a]);
            codes[a] = (const STRIX_CONSTANT u32x16*)(img.codes + static_cast<size_t>(r) * img.width);
            deltas[a] = img.deltas + static_cast<size_t>(r) * groups;
            sums[a] = img.sums + static_cast<size_t>(r) * groups;
        }
    }
};

__device__ __forceinline__ float lane_value(float v, uint32_t lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), static_cast<int>(lane)));
}

// One super-block (index kb along K, `blocks` in the row) of the lane's row, from ring slot `slot`, against the NA
// activation rows. The work is cut into 2 NA steps (activation row a, pair half); the codes of a step (two scalar
// loads of 64 bytes: n0, n1) are requested one step ahead, so on entry n0 / n1 hold step (kb, 0, 0) and on exit step
// (kb + 1, 0, 0). Scalar loads return out of order, so the only usable wait is "all of them": each step first waits for
// its own codes, then requests the next step's, then computes.
template <int NA>
__device__ __forceinline__ void block_compute(const uint8_t* slot, const ActRows<NA>& act, uint32_t kb, uint32_t blocks,
                                              const float (&vd)[NA], const float (&vf)[NA], u32x16& n0, u32x16& n1, float (&acc)[NA][4]) {
    const u32x4* blk = reinterpret_cast<const u32x4*>(slot + (threadIdx.x & 63U) * 144U);
    const u32x4 hd = blk[0];
    u32x4 q[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) q[i] = blk[1 + i];
    const float d = half_bits_to_float(hd.x & 0xffffU), dm = half_bits_to_float(hd.x >> 16);
    int lo[4][8], hi[4][8];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const uint32_t w[8] = {q[2 * p].x, q[2 * p].y, q[2 * p].z, q[2 * p].w, q[2 * p + 1].x, q[2 * p + 1].y, q[2 * p + 1].z, q[2 * p + 1].w};
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            lo[p][k] = static_cast<int>(w[k] & 0x0f0f0f0fU);
            hi[p][k] = static_cast<int>((w[k] >> 4) & 0x0f0f0f0fU);
        }
    }
    uint32_t sc[8], mn[8];
    q4k_factors<0>(hd, sc[0], mn[0]); q4k_factors<1>(hd, sc[1], mn[1]); q4k_factors<2>(hd, sc[2], mn[2]); q4k_factors<3>(hd, sc[3], mn[3]);
    q4k_factors<4>(hd, sc[4], mn[4]); q4k_factors<5>(hd, sc[5], mn[5]); q4k_factors<6>(hd, sc[6], mn[6]); q4k_factors<7>(hd, sc[7], mn[7]);
    float D[8], M[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        D[j] = d * static_cast<float>(sc[j]);
        M[j] = dm * static_cast<float>(mn[j]);
    }
    const uint32_t next_kb = kb + 1U < blocks ? kb + 1U : kb;      // the last block re-requests itself (unused)
    const uint32_t g0 = (kb & 7U) * 8U;
#pragma unroll
    for (int a = 0; a < NA; ++a) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            __builtin_amdgcn_s_waitcnt(0xC07F);                    // lgkmcnt(0): this step's codes have arrived
            const u32x16 c0 = n0, c1 = n1;
            __builtin_amdgcn_sched_barrier(0);
            {
                const int na = half ? (a + 1 < NA ? a + 1 : 0) : a;
                const uint32_t nb = (half && a + 1 == NA) ? next_kb : kb;
                const STRIX_CONSTANT u32x16* next = act.codes[na] + (nb * 4U + (half ? 0U : 2U));
                n0 = next[0];
                n1 = next[1];
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int pp = 0; pp < 2; ++pp) {
                const int p = 2 * half + pp;
                const u32x16& c = pp ? c1 : c0;
                int dot0 = 0, dot1 = 0;
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    dot0 = __builtin_amdgcn_sdot4(lo[p][k], static_cast<int>(c[k]), dot0, false);
                    dot1 = __builtin_amdgcn_sdot4(hi[p][k], static_cast<int>(c[8 + k]), dot1, false);
                }
                const float e0 = lane_value(vd[a], g0 + 2U * p), e1 = lane_value(vd[a], g0 + 2U * p + 1U);
                const float f0 = lane_value(vf[a], g0 + 2U * p), f1 = lane_value(vf[a], g0 + 2U * p + 1U);
                const float u0 = D[2 * p] * static_cast<float>(dot0), v0 = M[2 * p] * f0;
                const float u1 = D[2 * p + 1] * static_cast<float>(dot1), v1 = M[2 * p + 1] * f1;
                const float t0 = u0 - v0, t1 = u1 - v1;
                const float x0 = e0 * t0, x1 = e1 * t1;
                acc[a][p] = acc[a][p] + (x0 + x1);
            }
        }
    }
}

// Whole sweep: K = blocks super-blocks of the 64 rows described by `source` against the NA rows of `act`.
// value[a] = the lane's row against activation row a. `slots` are DEPTH separate LDS buffers of kStageBytes.
// On entry nothing is in flight; on exit every copy has landed and been consumed.
template <int NA, int DEPTH>
__device__ __forceinline__ void sweep_rows(uint8_t* const (&slots)[DEPTH], StageSource source, uint32_t blocks,
                                           const ActRows<NA>& act, float (&value)[NA]) {
    const uint32_t lane = threadIdx.x & 63U;
    float acc[NA][4];
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
        for (int p = 0; p < 4; ++p) acc[a][p] = 0.0F;
    float vd[NA], vf[NA];
#pragma unroll
    for (int a = 0; a < NA; ++a) vd[a] = vf[a] = 0.0F;
#pragma unroll
    for (int s = 0; s < DEPTH - 1; ++s)
        if (static_cast<uint32_t>(s) < blocks) source.start(slots[s]);
    u32x16 n0 = act.codes[0][0], n1 = act.codes[0][1];
    for (uint32_t b0 = 0; b0 < blocks; b0 += DEPTH) {
#pragma unroll
        for (int s = 0; s < DEPTH; ++s) {
            const uint32_t b = b0 + s;
            if (b < blocks) {
                if ((b & 7U) == 0) {           // refill the per-lane group deltas / sums: groups 8 b .. 8 b + 63
                    const uint32_t g = b * 8U + lane;
#pragma unroll
                    for (int a = 0; a < NA; ++a) {
                        vd[a] = g < act.groups ? act.deltas[a][g] : 0.0F;
                        vf[a] = g < act.groups ? static_cast<float>(act.sums[a][g]) : 0.0F;
                    }
                }
                // started so far: stages 0 .. min(blocks, b + DEPTH - 1) - 1; stage b must have landed
                const uint32_t last = b + DEPTH - 1U < blocks ? b + DEPTH - 1U : blocks;
                wait_stages_ahead(last - 1U - b);
                if (b + DEPTH - 1U < blocks) source.start(slots[(s + DEPTH - 1) % DEPTH]);
                block_compute<NA>(slots[s], act, b, blocks, vd, vf, n0, n1, acc);
            }
        }
    }
#pragma unroll
    for (int a = 0; a < NA; ++a) value[a] = (acc[a][0] + acc[a][1]) + (acc[a][2] + acc[a][3]);
}

}  // namespace strix950
