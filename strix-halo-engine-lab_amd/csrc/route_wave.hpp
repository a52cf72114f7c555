// Router for gfx950: logits, softmax, top-k, weights - and, for decode-sized batches, the A8 prologue and the expert
// plan in the same launch.
//
// Logits keep the reference's per-(row, expert) ascending fma chain (2048+ dependent fmas: latency, not bandwidth), so
// the chains are spread one wavefront per workgroup: a wave owns 8 experts x 8 rows (lane = 8 * expert + row), streams
// the router weight and the activations through LDS in 256-feature tiles (row-major, coalesced 128-bit loads, the next
// tile's loads in flight during the current tile's chain) and every lane reads its two operands with 128-bit LDS loads.
// Reference: tests/hip_moe_route_launcher_tests.hip:281-330 (chain), include/strix/moe/route_policy.hpp:99-156
// (softmax, selection, weights), src/hip_moe_route_launcher.hip:383-430 (chain kept per expert in the tiled kernel).
#pragma once
#include "device_math.hpp"

namespace strix950 {

constexpr uint32_t kRoutePass = 2048;         // features resident in LDS per pass (router weight slab + activation slab)
constexpr uint32_t kRouteMaxHidden = 16384, kRouteMaxExperts = 1024, kRouteMaxTopK = 16;
constexpr uint32_t kFusedMaxRows = 16;        // decode batches: router + prologue + plan in one launch

constexpr uint32_t kRouteRowPitch = kRoutePass + 4;   // floats; +16 bytes keeps the 8 rows of a slab on different banks
struct RouteLds {
    union {
        struct { float w[8][kRouteRowPitch]; float x[8][kRouteRowPitch]; } slab;   // 131,328 bytes: one pass of 8 expert rows + 8 activation rows
        struct { float p[8][kRouteMaxExperts + 1]; } sel;             // 32,800 bytes
        struct { uint32_t count[kRouteMaxExperts + 64]; } plan;
    };
    uint32_t ids[kFusedMaxRows * kRouteMaxTopK];    // selected experts of a decode batch, [row][top_k]
    float picked[8 * kRouteMaxTopK];                // selected scores of the 8 rows in flight, [row][k]
    uint32_t is_last;
};

struct RouteArgs {
    mi355_route_policy p;
    const uint8_t* x; uint32_t kind; uint64_t x_stride; uint32_t rows, hidden;
    const float* wr; const float* bias;
    uint32_t* ids; float* weights; float* scores;
    // fused decode extras (all null / zero for the plain router)
    int8_t* codes; float* deltas; int32_t* sums; uint32_t* status; uint32_t* job_status; uint32_t* plan;
    uint32_t route_blocks, quant_blocks;
};

// ---------------------------------------------------------------------------------------------------- logit chains
// Logits of 8 experts x 8 rows -> scores[row][expert] (used as the logit workspace). hidden % 32 == 0.
// Per pass of up to 2048 features: the 8 router-weight rows go global -> LDS by global_load_lds_dwordx4 (1 KiB of one row
// per instruction, nothing held in registers), the 8 activation rows are loaded, widened to fp32 once and stored to LDS;
// then every lane runs its chain reading both operands with 128-bit LDS loads at immediate offsets.
template <int KIND>
__device__ __forceinline__ void route_logits_block(RouteLds& lds, const RouteArgs& a, uint32_t e0, uint32_t r0) {
    const uint32_t lane = threadIdx.x, el = lane >> 3, t = lane & 7U;
    const bool butterfly = a.p.logits_order == MI355_LOGITS_LANE32_BUTTERFLY;
    float acc = 0.0F;
    float lanes32[32];
#pragma unroll
    for (int l = 0; l < 32; ++l) lanes32[l] = 0.0F;
    for (uint32_t k0 = 0; k0 < a.hidden; k0 += kRoutePass) {
        const uint32_t kc = a.hidden - k0 < kRoutePass ? a.hidden - k0 : kRoutePass;
        __syncthreads();
        // router weight rows: 16-byte piece `lane + 64 j` of row i
        for (uint32_t i = 0; i < 8U; ++i) {
            const uint32_t e = e0 + i < a.p.experts ? e0 + i : a.p.experts - 1U;
            const float* src = a.wr + static_cast<size_t>(e) * a.hidden + k0;
            for (uint32_t c0 = 0; c0 < kc / 4U; c0 += 64U)
                if (c0 + lane < kc / 4U)
                    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + 4U * (c0 + lane)),
                                                     (__attribute__((address_space(3))) void*)(&lds.slab.w[i][4U * c0]), 16, 0, 0);
        }
        // activation rows: 8 elements per lane and step, widened to fp32; one row's loads are all in flight together
        for (uint32_t i = 0; i < 8U; ++i) {
            const uint32_t r = r0 + i < a.rows ? r0 + i : a.rows - 1U;
            const uint8_t* src = a.x + r * a.x_stride + static_cast<size_t>(k0) * (KIND == 0 ? 4U : 2U);
            constexpr uint32_t steps = kRoutePass / 512U;
            if constexpr (KIND == 0) {
                f32x4 v[2 * steps];
#pragma unroll
                for (uint32_t j = 0; j < steps; ++j) {
                    const uint32_t c = 8U * lane + 512U * j, cc = c < kc ? c : 0U;
                    v[2 * j] = *reinterpret_cast<const f32x4*>(src + 4U * cc); v[2 * j + 1] = *reinterpret_cast<const f32x4*>(src + 4U * cc + 16U);
                }
#pragma unroll
                for (uint32_t j = 0; j < steps; ++j) {
                    const uint32_t c = 8U * lane + 512U * j;
                    if (c < kc) { *reinterpret_cast<f32x4*>(&lds.slab.x[i][c]) = v[2 * j]; *reinterpret_cast<f32x4*>(&lds.slab.x[i][c + 4U]) = v[2 * j + 1]; }
                }
            } else {
                u32x4 v[steps];
#pragma unroll
                for (uint32_t j = 0; j < steps; ++j) {
                    const uint32_t c = 8U * lane + 512U * j, cc = c < kc ? c : 0U;
                    v[j] = *reinterpret_cast<const u32x4*>(src + 2U * cc);
                }
#pragma unroll
                for (uint32_t j = 0; j < steps; ++j) {
                    const uint32_t c = 8U * lane + 512U * j;
                    const uint32_t h[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
                    float f[8];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        if constexpr (KIND == 1) { f[2 * q] = half_bits_to_float(h[q] & 0xffffU); f[2 * q + 1] = half_bits_to_float(h[q] >> 16); }
                        else { f[2 * q] = f_of(h[q] << 16); f[2 * q + 1] = f_of(h[q] & 0xffff0000U); }
                    }
                    if (c < kc) {
                        *reinterpret_cast<f32x4*>(&lds.slab.x[i][c]) = f32x4{f[0], f[1], f[2], f[3]};
                        *reinterpret_cast<f32x4*>(&lds.slab.x[i][c + 4U]) = f32x4{f[4], f[5], f[6], f[7]};
                    }
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        const float* wrow = lds.slab.w[el];
        const float* xrow = lds.slab.x[t];
        f32x4 wv[8], xv[8], wn[8], xn[8];      // operands of 32 features, fetched one block ahead of the chain
#pragma unroll
        for (uint32_t i = 0; i < 8; ++i) { wv[i] = *reinterpret_cast<const f32x4*>(wrow + 4U * i); xv[i] = *reinterpret_cast<const f32x4*>(xrow + 4U * i); }
        for (uint32_t k = 0; k < kc; k += 32U) {
            const uint32_t kn = k + 32U < kc ? k + 32U : k;
#pragma unroll
            for (uint32_t i = 0; i < 8; ++i) { wn[i] = *reinterpret_cast<const f32x4*>(wrow + kn + 4U * i); xn[i] = *reinterpret_cast<const f32x4*>(xrow + kn + 4U * i); }
            if (!butterfly) {
#pragma unroll
                for (uint32_t i = 0; i < 8; ++i) {
                    acc = __builtin_fmaf(xv[i].x, wv[i].x, acc); acc = __builtin_fmaf(xv[i].y, wv[i].y, acc);
                    acc = __builtin_fmaf(xv[i].z, wv[i].z, acc); acc = __builtin_fmaf(xv[i].w, wv[i].w, acc);
                }
            } else {      // 32 strided partial sums (product then add), the butterfly after the last pass (src/ds41_moe.cpp:74-83)
#pragma unroll
                for (uint32_t i = 0; i < 8; ++i) {
                    lanes32[4 * i] = lanes32[4 * i] + wv[i].x * xv[i].x; lanes32[4 * i + 1] = lanes32[4 * i + 1] + wv[i].y * xv[i].y;
                    lanes32[4 * i + 2] = lanes32[4 * i + 2] + wv[i].z * xv[i].z; lanes32[4 * i + 3] = lanes32[4 * i + 3] + wv[i].w * xv[i].w;
                }
            }
#pragma unroll
            for (uint32_t i = 0; i < 8; ++i) { wv[i] = wn[i]; xv[i] = xn[i]; }
        }
    }
    if (butterfly) {
#pragma unroll
        for (int s = 16; s; s /= 2)
#pragma unroll
            for (int i = 0; i < s; ++i) lanes32[i] = lanes32[i] + lanes32[i + s];
        acc = lanes32[0];
    }
    const uint32_t e = e0 + el, r = r0 + t;
    if (e < a.p.experts && r < a.rows) a.scores[static_cast<size_t>(r) * a.p.experts + e] = a.bias ? acc + a.bias[e] : acc;
    __syncthreads();
}

// ---------------------------------------------------------------------------------------------------- softmax + top-k
// One wave, up to 8 rows [r0, r0 + n): logits are read from scores[row][expert]; scores, ids and weights are written.
// Selection: k passes; a pass takes the greatest remaining score, the lower id on ties - the result of the reference's
// ascending serial scan with "c > best" (include/strix/moe/route_policy.hpp:107-121). sel_ids (optional, LDS) receives the
// ids as [row - r0][top_k].
struct RouteSelLds { float p[8][kRouteMaxExperts + 1]; float picked[8 * kRouteMaxTopK]; };
__device__ __forceinline__ void route_select_rows(float (*sel_p)[kRouteMaxExperts + 1], float* picked_lds, const RouteArgs& a, uint32_t r0, uint32_t n, uint32_t* sel_ids) {
    const uint32_t lane = threadIdx.x, E = a.p.experts, K = a.p.top_k;
    // softmax numerators, 8 lanes per row (all rows at once): m = max over the row, p = exp(z - m)
    {
        const uint32_t r = lane >> 3, sub = lane & 7U, rr = r < n ? r : n - 1U;
        const float* z = a.scores + static_cast<size_t>(r0 + rr) * E;
        float m = -INFINITY;
        for (uint32_t e = sub; e < E; e += 8U) { const float v = z[e]; m = v > m ? v : m; }
        { float o = xor1_f(m); m = o > m ? o : m; o = xor2_f(m); m = o > m ? o : m; o = xor4_f(m); m = o > m ? o : m; }
        if (r < n)
            for (uint32_t e = sub; e < E; e += 8U) sel_p[r][e] = declared_exp(z[e] - m);
    }
    __syncthreads();
    // denominators: one lane per row adds its row in ascending expert order from 0
    float total = 1.0F;
    if (lane < n) {
        float s = 0.0F;
        uint32_t e = 0;
        for (; e + 16U <= E; e += 16U) {         // 16 values per trip keep the LDS reads ahead of the dependent adds
            float v[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) v[i] = sel_p[lane][e + i];
#pragma unroll
            for (int i = 0; i < 16; ++i) s = s + v[i];
        }
        for (; e < E; ++e) s = s + sel_p[lane][e];
        total = s;
    }
    for (uint32_t r = 0; r < n; ++r) {
        const float sum = __shfl(total, static_cast<int>(r));
        for (uint32_t e = lane; e < E; e += 64U) {
            const float s = sel_p[r][e] / sum;
            sel_p[r][e] = s;
            a.scores[static_cast<size_t>(r0 + r) * E + e] = s;
        }
    }
    __syncthreads();
    // top-k: 8 lanes per row; lane `sub` owns experts sub, sub + 8, ... (ascending). A taken score is replaced by -1
    // (scores are >= 0), so one pass is a plain arg-max with the lower id winning ties. The pass loop is not unrolled.
    const uint32_t r = lane >> 3, sub = lane & 7U;
    const bool live = r < n;
    float* p = sel_p[live ? r : 0U];
    constexpr uint32_t kInReg = 32;                    // scores per lane kept in registers (experts <= 256)
    const bool in_reg = E <= 8U * kInReg;
    float mine[kInReg];
    if (in_reg) {
#pragma unroll
        for (uint32_t i = 0; i < kInReg; ++i) mine[i] = sub + 8U * i < E ? p[sub + 8U * i] : -2.0F;
    }
    __syncthreads();
    float* picked = picked_lds;
    float sum = 0.0F;
#pragma unroll 1
    for (uint32_t k = 0; k < K; ++k) {
        float bv = -3.0F;
        uint32_t bi = 0xffffffffU;
        if (in_reg) {
#pragma unroll
            for (uint32_t i = 0; i < kInReg; ++i)
                if (mine[i] > bv) { bv = mine[i]; bi = sub + 8U * i; }
        } else {
            for (uint32_t e = sub; e < E; e += 8U) {
                const float c = p[e];
                if (c > bv) { bv = c; bi = e; }
            }
        }
        {   // arg-max over the row's 8 lanes by DPP (lane ^ 1, ^ 2, ^ 4)
            float ov = xor1_f(bv); uint32_t oi = static_cast<uint32_t>(xor1_i(static_cast<int>(bi)));
            if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
            ov = xor2_f(bv); oi = static_cast<uint32_t>(xor2_i(static_cast<int>(bi)));
            if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
            ov = xor4_f(bv); oi = static_cast<uint32_t>(xor4_i(static_cast<int>(bi)));
            if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
        }
        if ((bi & 7U) == sub) {                        // the owner retires the pick
            if (in_reg) {
#pragma unroll
                for (uint32_t i = 0; i < kInReg; ++i)
                    if (i == (bi >> 3)) mine[i] = -1.0F;
            } else if (live) {
                p[bi] = -1.0F;
            }
        }
        sum = sum + bv;                                // ((0 + s_0) + s_1) + ... in selection order
        if (live && sub == 0) {
            a.ids[static_cast<size_t>(r0 + r) * K + k] = bi;
            if (sel_ids) sel_ids[r * K + k] = bi;
            picked[r * kRouteMaxTopK + k] = bv;
        }
    }
    const float den = sum + a.p.renorm_eps;
    if (live && sub == 0)
        for (uint32_t k = 0; k < K; ++k) {
            const float v = picked[r * kRouteMaxTopK + k];
            a.weights[static_cast<size_t>(r0 + r) * K + k] = (a.p.renormalize ? v / den : v) * a.p.scale;
        }
    __syncthreads();
}

}  // namespace strix950
