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
    struct { float w[8][kRouteRowPitch]; float x[8][kRouteRowPitch]; } slab;   // 131,328 bytes: one pass of 8 expert rows + 8 activation rows
};

struct RouteArgs {
    mi355_route_policy p;
    const uint8_t* x; uint32_t kind; uint64_t x_stride; uint32_t rows, hidden;
    const float* wr; const float* bias;
    uint32_t* ids; float* weights; float* scores;
    // fused decode extras (all null / zero for the plain router)
    int8_t* codes; float* deltas; int32_t* sums; uint32_t* status; uint32_t* job_status; uint32_t* plan;
    uint32_t route_blocks, quant_blocks;
    // RMSNorm of the input rows inside the launch (norm_on): the router and the A8 image see y = (x * r) * norm_w, r = 1 / sqrt(mean(x^2) + eps)
    // in the declared order of src/cpu/core/reference.cpp:86-103; normed (optional) receives y as fp32 [rows][hidden]
    uint32_t norm_on; const float* norm_w; float norm_eps; float* normed;
    // early-routes form (route_early.hpp): one word per assignment - the count of finished projection waves in the low half, a
    // non-finite projection in bit 31 -, and a test knob that displaces the early logits so that the repair path runs
    uint32_t* awords; uint32_t early_perturb;
    float* early_logits; uint32_t early_stride;      // where the early logits of row i go: early_logits + i * early_stride (floats)
};

// r of one row by a 64-thread workgroup, bit for bit rmsnorm_f32_kernel: lane l of L = 256 (n >= 512) or 128 chains
// fma(x, x, a) over x[l], x[l + L], ...; the L partial sums are halved in LDS; thread t stands for lanes t, t + 64, ...
template <int KIND>
__device__ __forceinline__ float row_norm_factor(float* partial /* 256 floats of LDS */, const uint8_t* xrow, uint32_t n, float eps) {
    const uint32_t t = threadIdx.x & 63U, L = n >= 512U ? 256U : 128U;
    for (uint32_t l = t; l < L; l += 64U) {
        float a = 0.0F;
        for (uint32_t i = l; i < n; i += L) {
            const float v = load_activation<KIND>(xrow, i);
            a = __builtin_fmaf(v, v, a);
        }
        partial[l] = a;
    }
    for (uint32_t h = L / 2U; h > 0; h >>= 1) {
        __syncthreads();
        for (uint32_t l = t; l < h; l += 64U) partial[l] = partial[l] + partial[l + h];
    }
    __syncthreads();
    const float r = 1.0F / __builtin_sqrtf(partial[0] / static_cast<float>(n) + eps);
    __syncthreads();
    return r;
}

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

// ---------------------------------------------------------------------------------------------------- batch chains
// Logits of large batches (the ascending fma chain form): throughput, not latency. A 256-thread workgroup owns 64 rows x
// 64 experts; a lane runs 4 x 4 independent chains (rows lr + 8 i, experts lc + 8 j of its wave's 32 x 32 quarter), so
// sixteen fmas separate two steps of the same chain and every pair of 128-bit LDS reads feeds 16 fmas. The tiles of 64
// features (activations widened to fp32 once) are register-staged one step ahead and double-buffered in LDS.
constexpr uint32_t kBatchTile = 64, kBatchStep = 64, kBatchPitch = kBatchStep + 4;     // floats; +16 bytes spreads the rows over the banks
struct BatchTiles { float w[2][kBatchTile][kBatchPitch]; float x[2][kBatchTile][kBatchPitch]; };     // 69,632 bytes

template <int KIND>
__device__ __forceinline__ void route_batch_block(BatchTiles& lds, const RouteArgs& a, uint32_t r0, uint32_t e0) {
    const uint32_t t = threadIdx.x, lane = t & 63U, wave = t >> 6;
    const uint32_t lrow = t >> 2, quarter = t & 3U;                    // loader role: tile row t / 4, 16 features
    const uint32_t le = e0 + lrow < a.p.experts ? e0 + lrow : a.p.experts - 1U;
    const uint32_t lr = r0 + lrow < a.rows ? r0 + lrow : a.rows - 1U;
    const float* wsrc = a.wr + static_cast<size_t>(le) * a.hidden + 16U * quarter;
    const uint8_t* xsrc = a.x + lr * a.x_stride + (KIND == 0 ? 64U : 32U) * quarter;
    const uint32_t steps = (a.hidden + kBatchStep - 1U) / kBatchStep;
    f32x4 wreg[4];
    u32x4 xreg[KIND == 0 ? 4 : 2];
    auto fetch = [&](uint32_t s) {
        // the last step of a row whose length is 32 mod 64: quarters 2, 3 re-read valid features (never used)
        const uint32_t k = s * kBatchStep, back = (k + 16U * quarter + 16U <= a.hidden) ? 0U : 32U;
        const float* ws = wsrc + k - back;
#pragma unroll
        for (int i = 0; i < 4; ++i) wreg[i] = *reinterpret_cast<const f32x4*>(ws + 4 * i);
        const uint8_t* xs = xsrc + static_cast<size_t>(k - back) * (KIND == 0 ? 4U : 2U);
#pragma unroll
        for (int i = 0; i < (KIND == 0 ? 4 : 2); ++i) xreg[i] = *reinterpret_cast<const u32x4*>(xs + 16 * i);
    };
    auto stage = [&](uint32_t buf) {
        float* wd = &lds.w[buf][lrow][16U * quarter];
        float* xd = &lds.x[buf][lrow][16U * quarter];
#pragma unroll
        for (int i = 0; i < 4; ++i) *reinterpret_cast<f32x4*>(wd + 4 * i) = wreg[i];
        if constexpr (KIND == 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(xd + 4 * i) = xreg[i];
        } else {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const uint32_t h[4] = {xreg[i].x, xreg[i].y, xreg[i].z, xreg[i].w};
                float f[8];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    if constexpr (KIND == 1) { f[2 * q] = half_bits_to_float(h[q] & 0xffffU); f[2 * q + 1] = half_bits_to_float(h[q] >> 16); }
                    else { f[2 * q] = f_of(h[q] << 16); f[2 * q + 1] = f_of(h[q] & 0xffff0000U); }
                }
                *reinterpret_cast<f32x4*>(xd + 8 * i) = f32x4{f[0], f[1], f[2], f[3]};
                *reinterpret_cast<f32x4*>(xd + 8 * i + 4) = f32x4{f[4], f[5], f[6], f[7]};
            }
        }
    };
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.0F;
    const uint32_t qr = 32U * (wave >> 1) + (lane >> 3), qe = 32U * (wave & 1U) + (lane & 7U);     // the lane's first row / expert in the tile
    fetch(0);
    stage(0);
    __syncthreads();
    for (uint32_t s = 0; s < steps; ++s) {
        const uint32_t buf = s & 1U;
        if (s + 1U < steps) fetch(s + 1U);
        const uint32_t kc = a.hidden - s * kBatchStep < kBatchStep ? a.hidden - s * kBatchStep : kBatchStep;
        for (uint32_t k = 0; k < kc; k += 4U) {
            f32x4 xv[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) xv[i] = *reinterpret_cast<const f32x4*>(&lds.x[buf][qr + 8 * i][k]);
#pragma unroll
            for (int j = 0; j < 4; ++j) wv[j] = *reinterpret_cast<const f32x4*>(&lds.w[buf][qe + 8 * j][k]);
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_fmaf(xv[i][c], wv[j][c], acc[i][j]);
        }
        if (s + 1U < steps) stage(buf ^ 1U);
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t r = r0 + qr + 8U * i, e = e0 + qe + 8U * j;
            if (r < a.rows && e < a.p.experts) a.scores[static_cast<size_t>(r) * a.p.experts + e] = a.bias ? acc[i][j] + a.bias[e] : acc[i][j];
        }
}

// ---------------------------------------------------------------------------------------------------- decode chains
// Decode batches (rows <= 16): one wavefront per (row, 8 experts). The chain of `hidden` dependent fmas is the whole
// cost (about 6 cycles per step), so everything else is taken off its path: the 8 router-weight rows and the activation
// row stream global -> LDS by global_load_lds_dwordx4 in chunks of 512 features through a ring of 4 slots (three chunks
// in flight during a chunk's chain, waits counted with s_waitcnt vmcnt); fp16 / bf16 activations are widened to fp32 in
// LDS once per chunk (a widening fma, v_fma_mix_f32, more than doubles the latency of a chain step); a lane reads its
// operands 32 features ahead of the chain with 128-bit LDS loads (the activation read is a broadcast).
// Lanes 8..63 repeat lanes 0..7 (a chain gains nothing from idle lanes).
constexpr uint32_t kChainChunk = 512;                 // features per ring slot
constexpr uint32_t kChainPitch = kChainChunk + 4;     // floats; +16 bytes keeps the 8 weight rows on different banks
constexpr uint32_t kChainExperts = 8;
template <bool NORM>
struct __attribute__((aligned(16))) ChainSlotT {
    float w[kChainExperts][kChainPitch];
    float x[kChainChunk];                             // the row's features as fp32
    uint32_t raw[kChainChunk / 2];                    // fp16 / bf16 input as copied (unused for fp32 input)
    float nw[NORM ? kChainChunk : 4];                 // the norm weights of the chunk (fused RMSNorm only)
};
// Four slots of the plain form are 78,336 bytes: two one-wave workgroups fit a compute unit's 160 KB (with the norm weights: one).
template <int KIND, bool NORM = false> constexpr uint32_t chain_copies() { return 2U * kChainExperts + (KIND == 0 ? 2U : 1U) + (NORM ? 2U : 0U); }

// Start the copy of features [k0, k0 + 512) of 8 router-weight rows and of the activation row. Every chunk issues the
// same number of copy instructions (the waits count them): lanes past the end of the row re-fetch its last piece into
// slot positions that are never read.
template <int KIND, bool NORM = false>
__device__ __forceinline__ void chain_start(ChainSlotT<NORM>& slot, const RouteArgs& a, uint32_t row, uint32_t e0, uint32_t k0) {
    const uint32_t lane = threadIdx.x & 63U;
    if constexpr (NORM) {       // (a null norm weight is a unit scale: the router weights stand in and are not used)
        const float* nsrc = a.norm_w ? a.norm_w : a.wr;
#pragma unroll
        for (uint32_t j = 0; j < 2U; ++j) {
            const uint32_t k = k0 + 256U * j + 4U * lane, kk = k + 4U <= a.hidden ? k : a.hidden - 4U;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(nsrc + kk),
                                             (__attribute__((address_space(3))) void*)(&slot.nw[256U * j]), 16, 0, 0);
        }
    }
#pragma unroll
    for (uint32_t i = 0; i < kChainExperts; ++i) {
        const uint32_t e = e0 + i < a.p.experts ? e0 + i : a.p.experts - 1U;
        const float* src = a.wr + static_cast<size_t>(e) * a.hidden;
#pragma unroll
        for (uint32_t j = 0; j < 2U; ++j) {
            const uint32_t k = k0 + 256U * j + 4U * lane, kk = k + 4U <= a.hidden ? k : a.hidden - 4U;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + kk),
                                             (__attribute__((address_space(3))) void*)(&slot.w[i][256U * j]), 16, 0, 0);
        }
    }
    const uint8_t* xrow = a.x + row * a.x_stride;
    if constexpr (KIND == 0) {
#pragma unroll
        for (uint32_t j = 0; j < 2U; ++j) {
            const uint32_t k = k0 + 256U * j + 4U * lane, kk = k + 4U <= a.hidden ? k : a.hidden - 4U;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(xrow + 4U * kk),
                                             (__attribute__((address_space(3))) void*)(&slot.x[256U * j]), 16, 0, 0);
        }
    } else {
        const uint32_t k = k0 + 8U * lane, kk = k + 8U <= a.hidden ? k : a.hidden - 8U;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(xrow + 2U * kk),
                                         (__attribute__((address_space(3))) void*)(&slot.raw[0]), 16, 0, 0);
    }
}
// fp16 / bf16: widen the landed chunk to fp32 (8 features per lane).
// The widened values are read by other lanes of the same wavefront (the workgroup is one wavefront): LDS operations of a
// wavefront complete in order, so the writes only have to be issued before the reads - no barrier. __syncthreads() here
// would also wait for every copy in flight, i.e. drain the three chunks the ring keeps ahead of the chain.
__device__ __forceinline__ void chain_publish() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
template <int KIND, bool NORM = false>
__device__ __forceinline__ void chain_widen(ChainSlotT<NORM>& slot, float factor = 1.0F, bool scaled = false) {
    if constexpr (KIND == 0 && NORM) {
        // fp32 rows arrive as they are: scale them in place, y = (x * r) * w
        const uint32_t lane = threadIdx.x & 63U;
#pragma unroll
        for (uint32_t j = 0; j < 2U; ++j) {
            f32x4 v = *reinterpret_cast<const f32x4*>(&slot.x[256U * j + 4U * lane]);
            const f32x4 w = *reinterpret_cast<const f32x4*>(&slot.nw[256U * j + 4U * lane]);
            v.x = v.x * factor; v.y = v.y * factor; v.z = v.z * factor; v.w = v.w * factor;
            if (scaled) { v.x = v.x * w.x; v.y = v.y * w.y; v.z = v.z * w.z; v.w = v.w * w.w; }
            *reinterpret_cast<f32x4*>(&slot.x[256U * j + 4U * lane]) = v;
        }
        chain_publish();
    }
    if constexpr (KIND != 0) {
        const uint32_t lane = threadIdx.x & 63U;
        const u32x4 r = *reinterpret_cast<const u32x4*>(&slot.raw[4U * lane]);
        const uint32_t h[4] = {r.x, r.y, r.z, r.w};
        float f[8];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if constexpr (KIND == 1) { f[2 * q] = half_bits_to_float(h[q] & 0xffffU); f[2 * q + 1] = half_bits_to_float(h[q] >> 16); }
            else { f[2 * q] = f_of(h[q] << 16); f[2 * q + 1] = f_of(h[q] & 0xffff0000U); }
        }
        if constexpr (NORM) {
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                f[q] = f[q] * factor;
                if (scaled) f[q] = f[q] * slot.nw[8U * lane + q];
            }
        }
        *reinterpret_cast<f32x4*>(&slot.x[8U * lane]) = f32x4{f[0], f[1], f[2], f[3]};
        *reinterpret_cast<f32x4*>(&slot.x[8U * lane + 4U]) = f32x4{f[4], f[5], f[6], f[7]};
        chain_publish();
    }
}

// Operands of 16 features: four 128-bit LDS reads of the lane's weight row and one 32-bit read that leaves feature k + t
// in lane t of every row of 16 lanes; the fma takes its activation operand from there by a row broadcast (a DPP operand,
// no instruction of its own). Measured on MI355X a wave pays ~5 cycles per dependent fma and ~9 per ds_read_b128, with no
// overlap between them; the operands of the next 16 features are requested before the current 16 are chained.
struct ChainStep { f32x4 w[4]; float x; };
template <bool NORM>
__device__ __forceinline__ void chain_load(ChainStep& s, const ChainSlotT<NORM>& slot, uint32_t el, uint32_t k) {
    const float* wrow = slot.w[el] + k;
#pragma unroll
    for (uint32_t i = 0; i < 4U; ++i) s.w[i] = *reinterpret_cast<const f32x4*>(wrow + 4U * i);
    s.x = slot.x[k + (threadIdx.x & 15U)];
}
// acc = fma(x[k + t], w[t], acc) for t = 0..15 in order. Written out as instructions because the compiler keeps the three-address
// fma, which has no DPP form, and then spends a v_mov_b32_dpp per feature. The leading s_nop covers the two wait states a DPP
// read needs after a vector-ALU write of its source register, whatever the compiler placed in front.
__device__ __forceinline__ float chain_run(const ChainStep& s, float acc) {
    asm("s_nop 1\n\t"
        "v_fmac_f32_dpp %0, %1, %2 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %3 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %4 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %5 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %6 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %7 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %8 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %9 row_newbcast:7 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %10 row_newbcast:8 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %11 row_newbcast:9 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %12 row_newbcast:10 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %13 row_newbcast:11 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %14 row_newbcast:12 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %15 row_newbcast:13 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %16 row_newbcast:14 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %17 row_newbcast:15 row_mask:0xf bank_mask:0xf"
        : "+v"(acc)
        : "v"(s.x), "v"(s.w[0].x), "v"(s.w[0].y), "v"(s.w[0].z), "v"(s.w[0].w), "v"(s.w[1].x), "v"(s.w[1].y), "v"(s.w[1].z), "v"(s.w[1].w),
          "v"(s.w[2].x), "v"(s.w[2].y), "v"(s.w[2].z), "v"(s.w[2].w), "v"(s.w[3].x), "v"(s.w[3].y), "v"(s.w[3].z), "v"(s.w[3].w));
    return acc;
}

template <int N>
__device__ __forceinline__ void chain_wait() { __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (0 << 8)); }      // (and every LDS read returned: the next copy reuses a slot this wave has read)

// Logits of experts [e0, e0 + 8) for one row -> scores[row][expert] (+ bias), stored for readers in other workgroups of
// the same launch. hidden % 32 == 0. slots: 4 separate LDS objects.
template <int KIND, bool NORM = false>
__device__ __forceinline__ void route_chain_block(ChainSlotT<NORM>* const (&slots)[4], const RouteArgs& a, uint32_t row, uint32_t e0, float r = 1.0F) {
    constexpr uint32_t NI = chain_copies<KIND, NORM>();
    const uint32_t lane = threadIdx.x & 63U, chunks = (a.hidden + kChainChunk - 1U) / kChainChunk;
    const bool butterfly = a.p.logits_order == MI355_LOGITS_LANE32_BUTTERFLY;
    const uint32_t el = lane & 7U;                      // chain form: the lane's expert
    const uint32_t bh = lane >> 5, bl = lane & 31U;     // butterfly form: experts bh, bh + 2, bh + 4, bh + 6; partial sum bl
    float acc = 0.0F, part[4] = {0.0F, 0.0F, 0.0F, 0.0F};
    chain_publish();      // a caller may have used slot memory as scratch (the norm factor): those LDS operations are complete before any copy
#pragma unroll
    for (uint32_t s = 0; s < 3U; ++s)
        if (s < chunks) chain_start<KIND, NORM>(*slots[s], a, row, e0, s * kChainChunk);
    for (uint32_t c0 = 0; c0 < chunks; c0 += 4U) {
#pragma unroll
        for (uint32_t s = 0; s < 4U; ++s) {
            const uint32_t c = c0 + s;
            if (c < chunks) {
                const uint32_t last = c + 3U < chunks ? c + 3U : chunks;       // chunks started so far: 0 .. last - 1
                const uint32_t ahead = last - 1U - c;
                if (ahead == 0) chain_wait<0>();
                else if (ahead == 1) chain_wait<NI>();
                else chain_wait<2 * NI>();
                if (c + 3U < chunks) chain_start<KIND, NORM>(*slots[(s + 3U) % 4U], a, row, e0, (c + 3U) * kChainChunk);
                ChainSlotT<NORM>& slot = *slots[s];
                chain_widen<KIND, NORM>(slot, r, a.norm_w != nullptr);
                const uint32_t kc = a.hidden - c * kChainChunk < kChainChunk ? a.hidden - c * kChainChunk : kChainChunk;
                if (!butterfly) {
                    if (kc == kChainChunk) {      // full chunk: straight-line code, operands fetched 16 features ahead
                        ChainStep A, B;
                        chain_load(A, slot, el, 0);
#pragma unroll
                        for (uint32_t k = 0; k < kChainChunk; k += 32U) {     // the barriers pin "fetch next, then chain"
                            chain_load(B, slot, el, k + 16U);
                            __builtin_amdgcn_sched_barrier(0);
                            acc = chain_run(A, acc);
                            __builtin_amdgcn_sched_barrier(0);
                            if (k + 32U < kChainChunk) chain_load(A, slot, el, k + 32U);
                            __builtin_amdgcn_sched_barrier(0);
                            acc = chain_run(B, acc);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    } else {                      // the last, partial chunk of the row
                        for (uint32_t k = 0; k < kc; k += 16U) {
                            ChainStep S;
                            chain_load(S, slot, el, k);
                            acc = chain_run(S, acc);
                        }
                    }
                } else {      // 32 strided partial sums per expert (product, then add); src/ds41_moe.cpp:74-83
                    for (uint32_t k = 0; k < kc; k += 32U) {
                        const float xv = slot.x[k + bl];
#pragma unroll
                        for (uint32_t j = 0; j < 4U; ++j) part[j] = part[j] + slot.w[bh + 2U * j][k + bl] * xv;
                    }
                }
            }
        }
    }
    float* out = a.scores + static_cast<size_t>(row) * a.p.experts;
    if (!butterfly) {
        const uint32_t e = e0 + el;
        if (lane < kChainExperts && e < a.p.experts)
            __hip_atomic_store(out + e, a.bias ? acc + a.bias[e] : acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
#pragma unroll
        for (uint32_t j = 0; j < 4U; ++j) {
            float v = part[j];
            v = v + xor16_f(v); v = v + xor8_f(v); v = v + xor4_f(v); v = v + xor2_f(v); v = v + xor1_f(v);
            const uint32_t e = e0 + bh + 2U * j;
            if (bl == 0 && e < a.p.experts)
                __hip_atomic_store(out + e, a.bias ? v + a.bias[e] : v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// ---------------------------------------------------------------------------------------------------- softmax + top-k (one row)
// One wave, one row: logits are read from scores[row][expert]; scores, ids and weights are written. Lane l owns experts
// l, l + 64, ... in registers (PER of them). Selection: k passes; a pass takes the greatest remaining score, the lower id
// on ties - the result of the reference's ascending serial scan with "c > best"
// (include/strix/moe/route_policy.hpp:107-121). A pass is one wave-wide maximum of 64-bit keys
// (score bits + 1) << 32 | ~id (scores are >= 0, so their bit patterns order like the values; 0 = taken or absent), reduced
// with DPP row shifts and row broadcasts into lane 63 and read back as a scalar. p_lds: kRouteMaxExperts floats.
__device__ __forceinline__ float max64(float v) {
    v = __builtin_fmaxf(v, xor1_f(v)); v = __builtin_fmaxf(v, xor2_f(v)); v = __builtin_fmaxf(v, xor4_f(v));
    v = __builtin_fmaxf(v, xor8_f(v)); v = __builtin_fmaxf(v, xor16_f(v)); v = __builtin_fmaxf(v, __shfl_xor(v, 32));
    return v;
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint64_t key_max_step(uint64_t key) {
    const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(static_cast<uint32_t>(key)), CTRL, ROW_MASK, 0xF, false));
    const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(static_cast<uint32_t>(key >> 32)), CTRL, ROW_MASK, 0xF, false));
    const uint64_t other = (static_cast<uint64_t>(hi) << 32) | lo;
    return other > key ? other : key;
}
__device__ __forceinline__ uint64_t key_max_wave(uint64_t key) {        // the wave's maximum, as a wave-uniform value
    key = key_max_step<0x111, 0xF>(key);      // row_shr:1
    key = key_max_step<0x112, 0xF>(key);      // row_shr:2
    key = key_max_step<0x114, 0xF>(key);      // row_shr:4
    key = key_max_step<0x118, 0xF>(key);      // row_shr:8   -> lane 15 of every row holds its row's maximum
    key = key_max_step<0x142, 0xA>(key);      // row_bcast:15 into rows 1 and 3
    key = key_max_step<0x143, 0xC>(key);      // row_bcast:31 into rows 2 and 3 -> lane 63 holds the wave's maximum
    const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(key)), 63));
    const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(key >> 32)), 63));
    return (static_cast<uint64_t>(hi) << 32) | lo;
}
// Returns, in lane k < top_k + shared_experts, the expert of slot k.
// shared_out: ids and weights are also read by other workgroups of the same launch (device-scope stores).
template <uint32_t PER>
__device__ __forceinline__ uint32_t route_select_row_per(float* p_lds, const RouteArgs& a, uint32_t row, bool shared_out) {
    const uint32_t lane = threadIdx.x & 63U, E = a.p.experts, K = a.p.top_k, P = K + a.p.shared_experts;
    float* z = a.scores + static_cast<size_t>(row) * E;
    float v[PER];
    float m = -INFINITY;
#pragma unroll
    for (uint32_t i = 0; i < PER; ++i) {
        const uint32_t e = lane + 64U * i;
        v[i] = e < E ? __hip_atomic_load(z + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : -INFINITY;   // written by other workgroups of this launch
        m = v[i] > m ? v[i] : m;
    }
    m = max64(m);
#pragma unroll
    for (uint32_t i = 0; i < PER; ++i) {
        const uint32_t e = lane + 64U * i;
        if (e < E) p_lds[e] = exp_of(a.p.exp_kind, v[i] - m);
    }
    __syncthreads();
    // denominator: ascending expert order from 0, computed by every lane (LDS broadcast reads, 16 values fetched ahead)
    float total = 0.0F;
    {
        const uint32_t full = E & ~15U;
        f32x4 t[4], n[4];
        if (full) {
#pragma unroll
            for (int i = 0; i < 4; ++i) t[i] = *reinterpret_cast<const f32x4*>(p_lds + 4 * i);
        }
        for (uint32_t e = 0; e < full; e += 16U) {
            const uint32_t en = e + 16U < full ? e + 16U : e;
#pragma unroll
            for (int i = 0; i < 4; ++i) n[i] = *reinterpret_cast<const f32x4*>(p_lds + en + 4 * i);
#pragma unroll
            for (int i = 0; i < 4; ++i) { total = total + t[i].x; total = total + t[i].y; total = total + t[i].z; total = total + t[i].w; }
#pragma unroll
            for (int i = 0; i < 4; ++i) t[i] = n[i];
        }
        for (uint32_t e = full; e < E; ++e) total = total + p_lds[e];
    }
    uint64_t key[PER];
#pragma unroll
    for (uint32_t i = 0; i < PER; ++i) {
        const uint32_t e = lane + 64U * i;
        key[i] = 0;
        if (e < E) {
            const float s = p_lds[e] / total;
            z[e] = s;
            key[i] = (static_cast<uint64_t>(b_of(s) + 1U) << 32) | (~e);
        }
    }
    float sum = 0.0F, my_v = 0.0F;
    uint32_t my_id = 0;
#pragma unroll 1
    for (uint32_t k = 0; k < K; ++k) {
        uint64_t best = key[0];
#pragma unroll
        for (uint32_t i = 1; i < PER; ++i) best = key[i] > best ? key[i] : best;
        best = key_max_wave(best);
        const uint32_t bi = ~static_cast<uint32_t>(best);
        const float bv = f_of(static_cast<uint32_t>(best >> 32) - 1U);
#pragma unroll
        for (uint32_t i = 0; i < PER; ++i)
            if (lane + 64U * i == bi) key[i] = 0;       // the owner retires the pick
        sum = sum + bv;                                // ((0 + s_0) + s_1) + ... in selection order
        if (lane == k) { my_v = bv; my_id = bi; }
    }
    const float den = sum + a.p.renorm_eps;
    if (lane < K) {
        store_shared_or_plain(shared_out, a.ids + static_cast<size_t>(row) * P + lane, my_id);
        const bool renorm = a.p.renormalize && (K > 1U || a.p.renorm_single);      // include/strix/moe/route_policy.hpp:146
        store_shared_or_plain(shared_out, a.weights + static_cast<size_t>(row) * P + lane, (renorm ? my_v / den : my_v) * a.p.scale);
    } else if (lane < P) {      // the always-on experts behind the routed ones: ids experts .. experts + shared - 1, weight 1 or the given gate
        my_id = E + (lane - K);
        a.ids[static_cast<size_t>(row) * P + lane] = my_id;
        a.weights[static_cast<size_t>(row) * P + lane] = a.p.shared_slot_weights ? a.p.shared_slot_weights[static_cast<size_t>(row) * a.p.shared_experts + (lane - K)] : 1.0F;
    }
    __syncthreads();
    return my_id;
}
__device__ __forceinline__ uint32_t route_select_row(float* p_lds, const RouteArgs& a, uint32_t row, bool shared_out = false) {
    const uint32_t E = a.p.experts;
    if (E <= 128U) return route_select_row_per<2>(p_lds, a, row, shared_out);
    if (E <= 256U) return route_select_row_per<4>(p_lds, a, row, shared_out);
    if (E <= 512U) return route_select_row_per<8>(p_lds, a, row, shared_out);
    return route_select_row_per<16>(p_lds, a, row, shared_out);
}

}  // namespace strix950
