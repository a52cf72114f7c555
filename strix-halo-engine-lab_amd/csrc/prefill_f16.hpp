// Prefill form of the routed experts for gfx950: an expert-grouped GEMM on the matrix cores. This is the path's second
// arithmetic class (the reference's FAST forms, include/strix/cuda/qwen_moe.hpp:100-101 "bit-changing"): Q4_K weights are
// dequantised exactly as the block decoder does (src/ggml_dequant.cpp:119-130: (d * sc) * q - (dmin * m), two fp32
// roundings), split into two fp16 numbers (w_hi = fp16(w), w_lo = fp16(w - w_hi): together ~22 significant bits - a single
// fp16 weight alone costs ~3e-3 of the output rms, above the tolerance), and multiplied with fp16 activations by
// v_mfma_f32_32x32x16_f16 with fp32 accumulation (two MFMAs per operand pair).
// Its parity target is the exact-weight product (include/strix/ds41_layer.hpp:96-121) within the stated tolerance, not
// the integer-dot class's bits.
//
// Work decomposition: the expert plan cuts every expert's assignments into items of at most 128 rows. A 256-thread
// workgroup owns (item, 64 output features of gate AND up) or (item, 128 output features of down): a 128 x 128 tile of
// weight rows x tokens, K walked in steps of 64 (one pair of Q4_K sub-blocks: the 32 quant bytes whose low / high nibbles
// are sub-blocks 2p / 2p + 1). Per step every thread fetches 16 quant bytes + the block header of one weight row and 64
// bytes of one token row into registers (one step ahead of the arithmetic), dequantises its 32 weights and stores the
// tiles row-major [row][k] (pitch 144 bytes: conflict-free 128-bit reads) in LDS (weights hi, weights lo, tokens).
// The workgroup has 8 waves in two roles: waves 0-3 are the loaders just described, waves 4-7 each multiply a 64 x 64
// quarter of the tile (2 x 2 MFMA tiles: every operand read from LDS feeds two MFMAs; 32 MFMAs per step). Tile rows are
// ordered [gate 0-31, up 0-31, gate 32-63, up 32-63] so that a wave holds gate and up of the same features. The LDS tiles are double-buffered and there is one barrier per
// step, so the loaders prepare step s + 1 (VALU) while the multipliers run step s (matrix cores) on the same SIMDs.
//
// Weights are read from HBM once per (item, feature tile); with ~128 rows per item the arithmetic intensity is ~450
// flop per weight byte, above the machine balance, so the kernel is bound by the matrix cores and the dequantisation
// that feeds them.
#pragma once
#include "device_math.hpp"

namespace strix950 {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr uint32_t kPfTile = 128;                 // weight rows and tokens per workgroup tile
constexpr uint32_t kPfStep = 64;                  // K per step
constexpr uint32_t kPfPitch = 144;                // bytes per tile row: 64 halves + 16 bytes of padding
constexpr uint32_t kPfTileBytes = kPfTile * kPfPitch;   // 18,432

struct PrefillArgs {
    const uint8_t* wa; const uint8_t* wb;         // MODE 0: gate, up; MODE 1: down (wb unused)
    uint64_t expert_stride, row_stride;           // bytes
    uint32_t k;                                   // K = hidden (MODE 0) or ffn (MODE 1), multiple of 256
    uint32_t features;                            // ffn (MODE 0) or hidden (MODE 1)
    uint32_t top_k, exp_kind;
    const uint8_t* x; uint64_t x_stride;          // MODE 0: fp16 token rows (bytes); MODE 1: unused
    _Float16* h;                                  // [assignments in plan order][ffn] fp16: written by MODE 0, read by MODE 1
    float* rawdots;                               // MODE 1: [assignment][hidden]
    const uint32_t* plan; uint32_t experts, assignments;
    uint32_t* status; uint32_t* job_status;
};

__device__ __forceinline__ uint32_t pack_half2(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(float2v{a, b}, half2v));      // v_cvt_pk_f16_f32: round to nearest even
}

// Raw operands of one K step held in registers between their global loads and their use.
struct PfRaw { u32x4 hd, qs, x[4]; };

template <int MODE>
__global__ __launch_bounds__(512) void prefill_f16_kernel(PrefillArgs a, uint32_t items_at, uint32_t order_at) {
    __shared__ __attribute__((aligned(16))) uint8_t tile_a[2][2][kPfTileBytes];     // [buffer][0: w_hi, 1: w_lo]
    __shared__ __attribute__((aligned(16))) uint8_t tile_b[2][kPfTileBytes];
    const uint4 item = *reinterpret_cast<const uint4*>(a.plan + items_at + 4U * blockIdx.y);
    const uint32_t e = item.x, begin = item.y, count = item.z - item.y;
    if (count == 0) return;
    if (MODE == 1 && (*a.job_status & MI355_STATUS_NONFINITE_PROJECTION)) return;
    const uint32_t* order = a.plan + order_at;
    const bool loader = threadIdx.x < 256U;
    const uint32_t t = threadIdx.x & 255U, lane = t & 63U, wave = t >> 6;      // index within the role
    // loader role: thread t owns weight row t / 2 of the tile and token t / 2, half = which 16 quant bytes / 32 features
    const uint32_t lrow = t >> 1, half = t & 1U;
    const uint32_t m0 = blockIdx.x * (MODE == 0 ? 64U : 128U);
    const uint8_t* wbase = (MODE == 0 && (lrow & 32U)) ? a.wb : a.wa;
    const uint32_t wfeature = MODE == 0 ? 32U * (lrow >> 6) + (lrow & 31U) : lrow;
    const uint8_t* wrow = wbase + static_cast<size_t>(e) * a.expert_stride + static_cast<size_t>(m0 + wfeature) * a.row_stride;
    // token loads: 8 consecutive lanes fetch the 128 bytes of one token row's step (whole cache lines); a thread serves
    // tokens t / 8 + 32 i, i = 0..3
    const uint8_t* xrow[4];
#pragma unroll
    for (uint32_t i = 0; i < 4U; ++i) {
        const uint32_t token = (t >> 3) + 32U * i, tok = token < count ? token : count - 1U;
        if (MODE == 0) xrow[i] = a.x + static_cast<size_t>(order[begin + tok] / a.top_k) * a.x_stride + 16U * (t & 7U);
        else xrow[i] = reinterpret_cast<const uint8_t*>(a.h + static_cast<size_t>(begin + tok) * a.k) + 16U * (t & 7U);
    }
    const uint32_t steps = a.k / kPfStep;

    auto fetch = [&](uint32_t s, PfRaw& r) {
        const uint32_t kb = s >> 2, p = s & 3U;
        const uint8_t* blk = wrow + static_cast<size_t>(kb) * 144U;
        r.hd = *reinterpret_cast<const u32x4*>(blk);
        r.qs = *reinterpret_cast<const u32x4*>(blk + 16U + 32U * p + 16U * half);
#pragma unroll
        for (int i = 0; i < 4; ++i) r.x[i] = *reinterpret_cast<const u32x4*>(xrow[i] + static_cast<size_t>(s) * kPfStep * 2U);
    };
    auto stage = [&](uint32_t s, const PfRaw& r, uint32_t buf) {
        const uint32_t p = s & 3U, j0 = 2U * p, sh0 = 8U * (j0 & 3U), sh1 = sh0 + 8U;
        const uint32_t fa0 = (r.hd.y >> sh0) & 255U, fb0 = (r.hd.z >> sh0) & 255U, fc0 = (r.hd.w >> sh0) & 255U;
        const uint32_t fa1 = (r.hd.y >> sh1) & 255U, fb1 = (r.hd.z >> sh1) & 255U, fc1 = (r.hd.w >> sh1) & 255U;
        const bool low = p < 2U;                  // uniform: p is the same for the whole workgroup
        const uint32_t s0 = low ? (fa0 & 63U) : ((fc0 & 15U) | ((fa0 >> 6) << 4)), n0 = low ? (fb0 & 63U) : ((fc0 >> 4) | ((fb0 >> 6) << 4));
        const uint32_t s1 = low ? (fa1 & 63U) : ((fc1 & 15U) | ((fa1 >> 6) << 4)), n1 = low ? (fb1 & 63U) : ((fc1 >> 4) | ((fb1 >> 6) << 4));
        const float d = half_bits_to_float(r.hd.x & 0xffffU), dm = half_bits_to_float(r.hd.x >> 16);
        const float D0 = d * static_cast<float>(s0), M0 = dm * static_cast<float>(n0);
        const float D1 = d * static_cast<float>(s1), M1 = dm * static_cast<float>(n1);
        const uint32_t q[4] = {r.qs.x, r.qs.y, r.qs.z, r.qs.w};
        // value -> (fp16 hi, fp16 lo) packed pairs; lo = fp16(value - hi) is exact to ~2^-22 of the value
        uint32_t lo_hi[8], lo_lo[8], hi_hi[8], hi_lo[8];
        const auto split2 = [](float v0, float v1, uint32_t& hi2, uint32_t& lo2) {
            const half2v h = __builtin_convertvector(float2v{v0, v1}, half2v);
            hi2 = __builtin_bit_cast(uint32_t, h);
            lo2 = pack_half2(v0 - static_cast<float>(h.x), v1 - static_cast<float>(h.y));
        };
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w = q[i];
            const float l0 = D0 * static_cast<float>(w & 15U) - M0, l1 = D0 * static_cast<float>((w >> 8) & 15U) - M0;
            const float l2 = D0 * static_cast<float>((w >> 16) & 15U) - M0, l3 = D0 * static_cast<float>((w >> 24) & 15U) - M0;
            const float h0 = D1 * static_cast<float>((w >> 4) & 15U) - M1, h1 = D1 * static_cast<float>((w >> 12) & 15U) - M1;
            const float h2 = D1 * static_cast<float>((w >> 20) & 15U) - M1, h3 = D1 * static_cast<float>(w >> 28) - M1;
            split2(l0, l1, lo_hi[2 * i], lo_lo[2 * i]); split2(l2, l3, lo_hi[2 * i + 1], lo_lo[2 * i + 1]);
            split2(h0, h1, hi_hi[2 * i], hi_lo[2 * i]); split2(h2, h3, hi_hi[2 * i + 1], hi_lo[2 * i + 1]);
        }
        uint8_t* ah = tile_a[buf][0] + lrow * kPfPitch;
        uint8_t* al = tile_a[buf][1] + lrow * kPfPitch;
        *reinterpret_cast<u32x4*>(ah + 32U * half) = u32x4{lo_hi[0], lo_hi[1], lo_hi[2], lo_hi[3]};
        *reinterpret_cast<u32x4*>(ah + 32U * half + 16U) = u32x4{lo_hi[4], lo_hi[5], lo_hi[6], lo_hi[7]};
        *reinterpret_cast<u32x4*>(ah + 64U + 32U * half) = u32x4{hi_hi[0], hi_hi[1], hi_hi[2], hi_hi[3]};
        *reinterpret_cast<u32x4*>(ah + 64U + 32U * half + 16U) = u32x4{hi_hi[4], hi_hi[5], hi_hi[6], hi_hi[7]};
        *reinterpret_cast<u32x4*>(al + 32U * half) = u32x4{lo_lo[0], lo_lo[1], lo_lo[2], lo_lo[3]};
        *reinterpret_cast<u32x4*>(al + 32U * half + 16U) = u32x4{lo_lo[4], lo_lo[5], lo_lo[6], lo_lo[7]};
        *reinterpret_cast<u32x4*>(al + 64U + 32U * half) = u32x4{hi_lo[0], hi_lo[1], hi_lo[2], hi_lo[3]};
        *reinterpret_cast<u32x4*>(al + 64U + 32U * half + 16U) = u32x4{hi_lo[4], hi_lo[5], hi_lo[6], hi_lo[7]};
        uint8_t* br = tile_b[buf] + (t >> 3) * kPfPitch + 16U * (t & 7U);
#pragma unroll
        for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(br + 32 * i * kPfPitch) = r.x[i];
    };

    floatx16 acc[2][2];                           // [row tile][token tile] of the wave's 64 x 64 quarter
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int n = 0; n < 2; ++n)
#pragma unroll
            for (int j = 0; j < 16; ++j) acc[i][n][j] = 0.0F;
    const uint32_t wr = wave >> 1, wc = wave & 1U;

    const uint32_t arow = lane & 31U, kq = (lane >> 5) * 16U;     // MFMA operand role: row / token lane & 31, 8 halves at k = 8 (lane / 32)
    PfRaw raw;
    if (loader) {
        fetch(0, raw);
        stage(0, raw, 0);
        if (steps > 1U) fetch(1, raw);
    }
    __syncthreads();
    for (uint32_t s = 0; s < steps; ++s) {
        const uint32_t buf = s & 1U;
        if (loader) {
            if (s + 1U < steps) {
                stage(s + 1U, raw, buf ^ 1U);                 // operands fetched during the previous step
                if (s + 2U < steps) fetch(s + 2U, raw);       // in flight during the next step
            }
        } else {
            const uint8_t* ta = tile_a[buf][0] + (64U * wr + arow) * kPfPitch + kq;
            const uint8_t* tl = tile_a[buf][1] + (64U * wr + arow) * kPfPitch + kq;
            const uint8_t* tb = tile_b[buf] + (64U * wc + arow) * kPfPitch + kq;
#pragma unroll
            for (uint32_t ks = 0; ks < 4U; ++ks) {
                half8 b[2], wl[2], wh[2];
#pragma unroll
                for (uint32_t i = 0; i < 2U; ++i) {
                    b[i] = *reinterpret_cast<const half8*>(tb + i * 32U * kPfPitch + 32U * ks);
                    wl[i] = *reinterpret_cast<const half8*>(tl + i * 32U * kPfPitch + 32U * ks);
                    wh[i] = *reinterpret_cast<const half8*>(ta + i * 32U * kPfPitch + 32U * ks);
                }
                // low planes first: consecutive MFMAs never wait for each other's accumulator
#pragma unroll
                for (uint32_t i = 0; i < 2U; ++i)
#pragma unroll
                    for (uint32_t n = 0; n < 2U; ++n) acc[i][n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wl[i], b[n], acc[i][n], 0, 0, 0);
#pragma unroll
                for (uint32_t i = 0; i < 2U; ++i)
#pragma unroll
                    for (uint32_t n = 0; n < 2U; ++n) acc[i][n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wh[i], b[n], acc[i][n], 0, 0, 0);
            }
        }
        __syncthreads();
    }
    if (loader) return;

    // C layout of a 32 x 32 tile: lane holds token (lane & 31); register i is weight row 8 (i / 4) + 4 (lane / 32) + i % 4
#pragma unroll
    for (uint32_t nt = 0; nt < 2U; ++nt) {
        const uint32_t n = 64U * wc + 32U * nt + (lane & 31U);
        const bool live = n < count;
        if (MODE == 0) {
            bool bad = false;
#pragma unroll
            for (uint32_t i4 = 0; i4 < 4U; ++i4) {
                float hv[4];
#pragma unroll
                for (uint32_t j = 0; j < 4U; ++j) {
                    const float g = acc[0][nt][4 * i4 + j], u = acc[1][nt][4 * i4 + j];
                    hv[j] = (g / (1.0F + declared_exp(-g))) * u;
                    bad = bad || !(finite_f(g) && finite_f(u) && finite_f(hv[j]));
                }
                if (live) {
                    const uint32_t row = m0 + 32U * wr + 8U * i4 + 4U * (lane >> 5);
                    u32x2 packed = {pack_half2(hv[0], hv[1]), pack_half2(hv[2], hv[3])};
                    *reinterpret_cast<u32x2*>(a.h + static_cast<size_t>(begin + n) * a.features + row) = packed;
                }
            }
            if (live && bad) {
                atomicOr(&a.status[order[begin + n] / a.top_k], static_cast<uint32_t>(MI355_STATUS_NONFINITE_PROJECTION));
                atomicOr(a.job_status, static_cast<uint32_t>(MI355_STATUS_NONFINITE_PROJECTION));
            }
        } else if (live) {
            float* out = a.rawdots + static_cast<size_t>(order[begin + n]) * a.features + m0 + 64U * wr;
#pragma unroll
            for (uint32_t m = 0; m < 2U; ++m)
#pragma unroll
                for (uint32_t i4 = 0; i4 < 4U; ++i4)
                    *reinterpret_cast<f32x4*>(out + 32U * m + 8U * i4 + 4U * (lane >> 5)) =
                        f32x4{acc[m][nt][4 * i4], acc[m][nt][4 * i4 + 1], acc[m][nt][4 * i4 + 2], acc[m][nt][4 * i4 + 3]};
        }
    }
}

}  // namespace strix950
