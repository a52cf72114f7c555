// MI355X (gfx950, wave64) kernels and C ABI of the quantized weight-product path. See include/mi355_strix.h for the
// contract of every entry point; reference file:line citations are relative to the reference tree.
#include "mi355_strix.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <string>

#include "device_math.hpp"
#include "q4k_rows.hpp"
#include "q4k_blocks.hpp"
#include "q4k_pairs.hpp"
#include "q4k_mma.hpp"
#include "q4k_quads.hpp"
#include "down_groups.hpp"
#include "q5k_quads.hpp"
#include "q6k_quads.hpp"
#include "prefill_f16.hpp"
#include "prefill_reg.hpp"
#include "route_wave.hpp"
#include "route_early.hpp"

namespace strix950 {

// ======================================================================================================== host side
thread_local std::string g_error;

int32_t fail(int32_t code, const char* what) {
    g_error = what;
    return code;
}
int32_t hip_fail(hipError_t e, const char* what) {
    g_error = std::string(what) + ": " + hipGetErrorString(e);
    return MI355_E_HIP;
}
#define STRIX_REQUIRE(cond, what) do { if (!(cond)) return fail(MI355_E_INVALID_ARGUMENT, what); } while (0)
#define STRIX_LAUNCHED(what) do { const hipError_t e_ = hipGetLastError(); if (e_ != hipSuccess) return hip_fail(e_, what); } while (0)

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }
inline hipStream_t hs(mi355_stream s) { return static_cast<hipStream_t>(s); }

constexpr uint32_t kQ4kBlock = 144, kQ80Block = 34;

// ======================================================================================================== block decode
// One thread per output element. Q4_K: y = (d * sc) * q - (dmin * m), two products and one subtraction
// (src/ggml_dequant.cpp:119-130); Q8_0: y = int8 * d (src/ggml_dequant.cpp:84-87).
__device__ __forceinline__ void q4k_scale_min(const uint8_t* q, uint32_t j, uint32_t& sc, uint32_t& m) {
    if (j < 4) { sc = q[j] & 63U; m = q[j + 4] & 63U; }
    else { sc = (q[j + 4] & 0xFU) | ((q[j - 4] >> 6) << 4); m = (q[j + 4] >> 4) | ((q[j] >> 6) << 4); }
}

__global__ __launch_bounds__(256) void dequantize_rows_kernel(uint32_t type, const uint8_t* rows, uint64_t row_stride,
                                                              uint32_t elements, float* out, uint64_t out_stride) {
    const uint32_t r = blockIdx.y;
    const uint8_t* row = rows + r * row_stride;
    for (uint32_t i = blockIdx.x * 256U + threadIdx.x; i < elements; i += gridDim.x * 256U) {
        float y;
        if (type == MI355_TYPE_Q8_0) {
            const uint8_t* b = row + (i / 32U) * kQ80Block;
            const float d = half_bits_to_float(b[0] | (static_cast<uint32_t>(b[1]) << 8));
            y = static_cast<float>(static_cast<int8_t>(b[2 + (i % 32U)])) * d;
        } else {
            const uint8_t* b = row + (i / 256U) * kQ4kBlock;
            const uint32_t k = i % 256U, j = k / 32U, l = k % 32U;
            uint32_t sc, m;
            q4k_scale_min(b + 4, j, sc, m);
            const float d = half_bits_to_float(b[0] | (static_cast<uint32_t>(b[1]) << 8));
            const float mn = half_bits_to_float(b[2] | (static_cast<uint32_t>(b[3]) << 8));
            const float d1 = d * static_cast<float>(sc), m1 = mn * static_cast<float>(m);
            const uint32_t byte = b[16 + 32 * (j / 2) + l];
            const float q = static_cast<float>((j & 1U) ? (byte >> 4) : (byte & 15U));
            y = d1 * q - m1;
        }
        out[r * out_stride + i] = y;
    }
}

// ======================================================================================================== weight writers
// Q8_0: include/strix/q8_0_rule.hpp:25-33 (d = amax / 127, id = 1 / d, q = roundf(v * id), d stored as fp16).
__global__ __launch_bounds__(256) void quantize_q8_0_rows_kernel(const float* x, uint64_t blocks, uint8_t* out) {
    for (uint64_t b = blockIdx.x * 256ULL + threadIdx.x; b < blocks; b += 256ULL * gridDim.x) {
        const float* v = x + b * 32;
        float amax = 0.0F;
        for (int j = 0; j < 32; ++j) amax = __builtin_fmaxf(amax, __builtin_fabsf(v[j]));
        const float d = amax / 127.0F;
        const float id = d != 0.0F ? 1.0F / d : 0.0F;
        uint8_t* o = out + b * kQ80Block;
        const uint32_t h = float_to_half_bits(d);
        o[0] = static_cast<uint8_t>(h); o[1] = static_cast<uint8_t>(h >> 8);
        for (int j = 0; j < 32; ++j) o[2 + j] = static_cast<uint8_t>(static_cast<int8_t>(static_cast<int>(__builtin_roundf(v[j] * id))));
    }
}

// Q4_K min/max writer (no reference counterpart; the reference only reads GGUF). Per 32-value sub-block: scale =
// (max - min) / 15 and offset = 0 - min with min clamped to <= 0; super-block d = max scale / 63, dmin = max offset / 63,
// both stored as fp16; 6-bit factors and 4-bit codes by round-to-nearest against the fp16-rounded d / dmin.
__global__ __launch_bounds__(64) void quantize_q4_k_rows_kernel(const float* x, uint64_t blocks, uint8_t* out) {
    for (uint64_t b = blockIdx.x * 64ULL + threadIdx.x; b < blocks; b += 64ULL * gridDim.x) {
        const float* v = x + b * 256;
        uint8_t* o = out + b * kQ4kBlock;
        float scale[8], offset[8], smax = 0.0F, omax = 0.0F;
        for (int j = 0; j < 8; ++j) {
            float lo = 0.0F, hi = v[32 * j];
            for (int l = 0; l < 32; ++l) { lo = __builtin_fminf(lo, v[32 * j + l]); hi = __builtin_fmaxf(hi, v[32 * j + l]); }
            hi = __builtin_fmaxf(hi, lo);
            scale[j] = (hi - lo) / 15.0F; offset[j] = 0.0F - lo;
            smax = __builtin_fmaxf(smax, scale[j]); omax = __builtin_fmaxf(omax, offset[j]);
        }
        const uint32_t dh = float_to_half_bits(smax / 63.0F), mh = float_to_half_bits(omax / 63.0F);
        const float d = half_bits_to_float(dh), dm = half_bits_to_float(mh);
        uint32_t sc[8], mn[8];
        for (int j = 0; j < 8; ++j) {
            sc[j] = d > 0.0F ? static_cast<uint32_t>(__builtin_fminf(63.0F, __builtin_rintf(scale[j] / d))) : 0U;
            mn[j] = dm > 0.0F ? static_cast<uint32_t>(__builtin_fminf(63.0F, __builtin_rintf(offset[j] / dm))) : 0U;
        }
        o[0] = static_cast<uint8_t>(dh); o[1] = static_cast<uint8_t>(dh >> 8);
        o[2] = static_cast<uint8_t>(mh); o[3] = static_cast<uint8_t>(mh >> 8);
        for (int j = 0; j < 4; ++j) {
            o[4 + j] = static_cast<uint8_t>((sc[j] & 63U) | ((sc[j + 4] >> 4) << 6));
            o[8 + j] = static_cast<uint8_t>((mn[j] & 63U) | ((mn[j + 4] >> 4) << 6));
            o[12 + j] = static_cast<uint8_t>((sc[j + 4] & 15U) | ((mn[j + 4] & 15U) << 4));
        }
        for (int p = 0; p < 4; ++p) {
            const float ed0 = d * static_cast<float>(sc[2 * p]), em0 = dm * static_cast<float>(mn[2 * p]);
            const float ed1 = d * static_cast<float>(sc[2 * p + 1]), em1 = dm * static_cast<float>(mn[2 * p + 1]);
            for (int l = 0; l < 32; ++l) {
                float r0 = 0.0F, r1 = 0.0F;
                if (ed0 > 0.0F) r0 = __builtin_fminf(15.0F, __builtin_fmaxf(0.0F, __builtin_rintf((v[64 * p + l] + em0) / ed0)));
                if (ed1 > 0.0F) r1 = __builtin_fminf(15.0F, __builtin_fmaxf(0.0F, __builtin_rintf((v[64 * p + 32 + l] + em1) / ed1)));
                o[16 + 32 * p + l] = static_cast<uint8_t>(static_cast<uint32_t>(r0) | (static_cast<uint32_t>(r1) << 4));
            }
        }
    }
}

// ======================================================================================================== A8 quantiser
// RMSNorm of fp32 rows in the reference's declared order (src/cpu/core/reference.cpp:86-103, lane count
// src/cpu/core/backend.hpp:91): lane l of L = 256 (n >= 512) or 128 runs the fma chain over x[l], x[l + L], ...; the L partial
// sums are halved in LDS (partial[l] += partial[l + h], h = L/2 .. 1); r = 1 / sqrt(sum / n + eps); y = (x * r) * w.
// One workgroup of L threads per row: the lanes' strided chains are coalesced reads as they stand.
__global__ __launch_bounds__(256) void rmsnorm_f32_kernel(const float* x, const float* w, uint32_t n, float eps, float* y) {
    __shared__ float partial[256];
    const uint32_t lanes = blockDim.x, lane = threadIdx.x;
    const float* xr = x + static_cast<size_t>(blockIdx.x) * n;
    float* yr = y + static_cast<size_t>(blockIdx.x) * n;
    float a = 0.0F;
    for (uint32_t i = lane; i < n; i += lanes) a = __builtin_fmaf(xr[i], xr[i], a);
    partial[lane] = a;
    for (uint32_t h = lanes / 2U; h > 0; h >>= 1) {
        __syncthreads();
        if (lane < h) partial[lane] = partial[lane] + partial[lane + h];
    }
    __syncthreads();
    const float r = 1.0F / __builtin_sqrtf(partial[0] / static_cast<float>(n) + eps);
    for (uint32_t i = lane; i < n; i += lanes) yr[i] = w ? (xr[i] * r) * w[i] : xr[i] * r;
}

// One aligned group of 32 lanes per 32-value group; 8 groups per 256-thread block.
// Reference: src/cpu/core/reference.cpp:35-55.
// nan_delta: the dense A8 profile's rule for a group that holds a non-finite value (src/hip_q8_rows_gemv.hpp:1157-1161,1232-1250): its
// delta is the canonical NaN 0x7fc00000 and its codes are 0, so that every product over the group is NaN.
template <int KIND>
__global__ __launch_bounds__(256) void quantize_a8_kernel(const uint8_t* x, uint64_t x_stride, uint32_t width, int8_t* codes,
                                                          float* deltas, int32_t* sums, uint32_t* status, uint32_t nan_delta = 0) {
    const uint32_t r = blockIdx.y, groups = width / 32U;
    const uint32_t g = blockIdx.x * 8U + (threadIdx.x >> 5), j = threadIdx.x & 31U;
    if (g >= groups) return;
    const float v = load_activation<KIND>(x + r * x_stride, g * 32U + j);
    const float amax = max32(__builtin_fabsf(v));
    const bool tiny = amax > 0.0F && amax < 0x1p-119F;
    const float delta = (amax == 0.0F || tiny) ? 1.0F : amax / 127.0F;
    const int bad = or32_i(finite_f(v) ? 0 : 1);
    const int code = (bad && nan_delta) ? 0 : a8_code(v, delta, tiny);
    const int sum = sum32_i(code);
    codes[static_cast<size_t>(r) * width + g * 32U + j] = static_cast<int8_t>(code);
    if (j == 0) {
        deltas[static_cast<size_t>(r) * groups + g] = (bad && nan_delta) ? __builtin_bit_cast(float, 0x7fc00000U) : delta;
        if (sums) sums[static_cast<size_t>(r) * groups + g] = sum;
        if (bad && status) atomicOr(&status[r], static_cast<uint32_t>(MI355_STATUS_NONFINITE_ACTIVATION));
    }
}

// ======================================================================================================== Q8_0 x A8 GEMV
// One aligned group of 32 lanes per output row: lane l owns the reference's accumulator lane l (groups g = l, l + 32,
// ... ascending), then the tree32 butterfly. Up to RB activation rows share one sweep of the weight row.
// Reference: src/cpu/core/reference.cpp:57-84, src/core/integer_math.hpp:11-13,43-47.
// DW: the weight rows are 4-byte aligned. A block (34 bytes: fp16 scale, 32 codes) is then fetched as nine aligned dwords
// (two 128-bit loads and one 32-bit load) around its codes and shifted into place, instead of seventeen 16-bit loads.
// CHAIN (RB = 1): the row contract of the reference's dense A8 profile (src/hip_q8_rows_gemv.hpp:1155-1170; host statement
// tests/dense_a8_small_reference_tests.cpp:93-104): acc = +0, then for the blocks in ascending order acc = fma(float(d_w) * delta,
// float(dot), acc), and a NaN result is stored as 0x7fc00000. The lanes evaluate their blocks as before and leave every block's
// (scale, dot) pair in LDS; lane 0 of the output's 32 lanes then walks them in order.
constexpr uint32_t kGemvChainMaxGroups = 256;          // in <= 8192 (kDenseA8MaxWidth, src/hip_q8_rows_gemv.hpp:1176)
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
template <int RB, bool DW, bool CHAIN = false>
__global__ __launch_bounds__(256) void gemv_q8_0_a8_kernel(mi355_q8a8_view v) {
    __shared__ float2 chain_pairs[CHAIN ? 8 : 1][CHAIN ? kGemvChainMaxGroups : 1];
    const uint32_t o = blockIdx.x * 8U + (threadIdx.x >> 5), l = threadIdx.x & 31U, row0 = blockIdx.y * RB;
    if (o >= v.count) return;
    const uint32_t groups = v.in / 32U;
    const uint32_t nr = v.rows - row0 < static_cast<uint32_t>(RB) ? v.rows - row0 : static_cast<uint32_t>(RB);
    const uint8_t* wrow = v.weight + static_cast<size_t>(o) * v.row_bytes;
    float lane[RB];
#pragma unroll
    for (int r = 0; r < RB; ++r) lane[r] = 0.0F;
    // (unrolled: the loads of four of the lane's groups are in flight together; the accumulation order does not change)
#pragma unroll 4
    for (uint32_t g = l; g < groups; g += 32U) {
        const unsigned short* b = reinterpret_cast<const unsigned short*>(wrow + static_cast<size_t>(g) * kQ80Block);
        const float scale = half_bits_to_float(b[0]);
        int w[8];
        if constexpr (DW) {
            const uint32_t c0 = g * kQ80Block + 2U, shift = c0 & 3U;          // first code byte: 0 or 2 past a dword boundary
            const uint32_t* dw = reinterpret_cast<const uint32_t*>(wrow) + (c0 >> 2);
            const u32x4_a4 lo4 = *reinterpret_cast<const u32x4_a4*>(dw), hi4 = *reinterpret_cast<const u32x4_a4*>(dw + 4);
            const uint32_t last = dw[shift ? 8 : 7];                          // (an aligned block ends with its eighth dword)
            const uint32_t d[9] = {lo4.x, lo4.y, lo4.z, lo4.w, hi4.x, hi4.y, hi4.z, hi4.w, last};
#pragma unroll
            for (int i = 0; i < 8; ++i) w[i] = static_cast<int>(__builtin_amdgcn_alignbyte(d[i + 1], d[i], shift));
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) w[i] = static_cast<int>(static_cast<uint32_t>(b[1 + 2 * i]) | (static_cast<uint32_t>(b[2 + 2 * i]) << 16));
        }
#pragma unroll
        for (int r = 0; r < RB; ++r) {
            if (static_cast<uint32_t>(r) < nr) {
                const int4* xc = reinterpret_cast<const int4*>(v.codes + static_cast<size_t>(row0 + r) * v.x_stride + g * 32U);
                const int4 a = xc[0], c = xc[1];
                int dot = 0;
                dot = __builtin_amdgcn_sdot4(w[0], a.x, dot, false); dot = __builtin_amdgcn_sdot4(w[1], a.y, dot, false);
                dot = __builtin_amdgcn_sdot4(w[2], a.z, dot, false); dot = __builtin_amdgcn_sdot4(w[3], a.w, dot, false);
                dot = __builtin_amdgcn_sdot4(w[4], c.x, dot, false); dot = __builtin_amdgcn_sdot4(w[5], c.y, dot, false);
                dot = __builtin_amdgcn_sdot4(w[6], c.z, dot, false); dot = __builtin_amdgcn_sdot4(w[7], c.w, dot, false);
                const float xd = v.deltas[static_cast<size_t>(row0 + r) * (v.x_stride / 32U) + g];
                if constexpr (CHAIN) chain_pairs[threadIdx.x >> 5][g] = make_float2(scale * xd, static_cast<float>(dot));
                else lane[r] = lane[r] + static_cast<float>(dot) * (scale * xd);
            }
        }
    }
    if constexpr (CHAIN) {
        // the pairs were written by lanes of this wave: program order of one wave's LDS accesses
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (l == 0) {
            float acc = 0.0F;
            for (uint32_t g = 0; g < groups; ++g) {
                const float2 c = chain_pairs[threadIdx.x >> 5][g];
                acc = __builtin_fmaf(c.x, c.y, acc);
            }
            v.out[static_cast<size_t>(row0) * v.out_stride + o] = acc != acc ? __builtin_bit_cast(float, 0x7fc00000U) : acc;
        }
        return;
    }
#pragma unroll
    for (int r = 0; r < RB; ++r) {
        float p = lane[r];
        p = p + xor16_f(p); p = p + xor8_f(p); p = p + xor4_f(p); p = p + xor2_f(p); p = p + xor1_f(p);
        if (l == 0 && static_cast<uint32_t>(r) < nr) {
            float* y = &v.out[static_cast<size_t>(row0 + r) * v.out_stride + o];
            *y = v.accumulate ? *y + p : p;
        }
    }
}

// ======================================================================================================== router
// Plan words (uint32): [0] assignments A = rows * top_k, [1] touched experts U, [2] largest group, [3] launch ticket,
// [4] work items; [16, 272) ticket / scratch words; offsets[experts + 1]; touched[experts] (ids of the experts with work,
// ascending); order[A]: assignment indices (row * top_k + slot) grouped by expert, ascending row then slot inside an
// expert; items[A] x 4 words {expert, begin, end, 0}: the work items of the expert kernels, a touched expert's assignments
// cut into pieces of at most `split` (zero records after the last item, up to the launch's item bound).
// Reference: src/hip_moe_q4k_a8_probe.hip:91-147 (stable CSR of (row, slot) by expert).
__host__ __device__ constexpr uint32_t pad4(uint32_t v) { return (v + 3U) & ~3U; }
// ticket / scratch words right after the header, at the same place for every batch size (every launch leaves them zero, and a
// workspace is reused with varying row counts): [0, 16) row tickets of the fused router, [16, 32) its quantiser tickets,
// [128, 144) per-row A8 flags of the fused prologue
constexpr uint32_t kPlanTicketsAt = 16, kPlanTicketWords = 256;
// Behind the ticket words, also at a fixed place, the words of a decode batch planned from early routes (route_early.hpp):
//   one word per assignment (finished projection waves in the low half, bit 31 = non-finite projection);
//   one 64-bit tag per assignment {epoch, early expert};
//   three 128-byte lines per row (arrival counts of the early blocks, of the A8 prologue blocks - with the row's flag word beside
//     it - and of the exact router's side blocks) and a line with one tag per row (epoch of the call whose A8 image of that row is
//     complete) and the epoch word.
// Counts are zero when the plan is allocated and every launch leaves them zero. The epoch of a call is the epoch word + 1; the
// call's down launch stores it back, so tags of earlier calls never look current and nothing has to be reset.
constexpr uint32_t kLineWords = 32, kEarlyMaxAssignments = 128, kEarlyMinAssignments = 8, kEarlyMaxRows = 16;
constexpr uint32_t kPlanAwordsAt = kPlanTicketsAt + kPlanTicketWords, kPlanEtagsAt = kPlanAwordsAt + kEarlyMaxAssignments;
constexpr uint32_t kPlanLinesAt = (kPlanEtagsAt + 2U * kEarlyMaxAssignments + kLineWords - 1U) / kLineWords * kLineWords;      // (lines of a 128-byte aligned plan)
constexpr uint32_t kLinesEarly = 0, kLinesPrologue = kEarlyMaxRows * kLineWords, kLinesSide = 2U * kEarlyMaxRows * kLineWords;
constexpr uint32_t kLinesRowTags = 3U * kEarlyMaxRows * kLineWords, kLinesEpoch = kLinesRowTags + kEarlyMaxRows;
constexpr uint32_t kPlanOffsetsAt = kPlanLinesAt + kLinesRowTags + kLineWords;
static_assert(kPlanEtagsAt % 2U == 0 && kPlanOffsetsAt % 4U == 0, "tags on 8 bytes, the plan arrays on 16");
__host__ __device__ constexpr uint32_t plan_touched_at(uint32_t experts) { return kPlanOffsetsAt + pad4(experts + 1U); }
__host__ __device__ constexpr uint32_t plan_order_at(uint32_t experts) { return plan_touched_at(experts) + pad4(experts); }
// most work items a plan can hold (layout) and most a launch with pieces of `split` assignments can produce (grid size)
__host__ __device__ constexpr uint32_t plan_item_capacity(uint32_t assignments) { return assignments; }
__host__ __device__ inline uint32_t plan_item_bound(uint32_t experts, uint32_t assignments, uint32_t split) {
    const uint32_t most = experts + assignments / split;
    return assignments < most ? assignments : most;
}
__host__ __device__ constexpr uint32_t plan_items_at(uint32_t experts, uint32_t assignments) { return plan_order_at(experts) + pad4(assignments); }
__host__ __device__ constexpr uint32_t plan_words_total(uint32_t experts, uint32_t assignments) {
    return plan_items_at(experts, assignments) + 4U * plan_item_capacity(assignments);
}

// Router logits for batches above the decode bound: blocks of 8 experts x 8 rows.
template <int KIND>
__global__ __launch_bounds__(64) void route_logits_kernel(RouteArgs a) {
    __shared__ RouteLds lds;
    const uint32_t neb = (a.p.experts + 7U) / 8U;
    route_logits_block<KIND>(lds, a, (blockIdx.x % neb) * 8U, (blockIdx.x / neb) * 8U);
}

// Router logits of large batches in the ascending fma chain order: 64 rows x 64 experts per 256-thread workgroup.
template <int KIND>
__global__ __launch_bounds__(256, 2) void route_batch_kernel(RouteArgs a) {
    __shared__ __attribute__((aligned(16))) BatchTiles lds;
    route_batch_block<KIND>(lds, a, blockIdx.y * kBatchTile, blockIdx.x * kBatchTile);
}

// A8 prologue block qb of a fused decode launch (src/cpu/core/reference.cpp:35-55): two groups of 32 at a time, 8 groups per
// block; the last of a row's blocks publishes the row's status word. scratch: 256 floats of LDS (fused RMSNorm only).
// Row r counts its finished blocks in ticket[r * stride] and collects its flags in flags[r * stride]. LINES: the words are reached
// by device-scope atomics only and the count is a plain arrival (route_early.hpp); otherwise the count is an acquire-release ticket.
template <int KIND, bool NORM, bool LINES = false>
__device__ __forceinline__ void a8_prologue_block(const RouteArgs& a, uint32_t qb, uint32_t* ticket, uint32_t* flags, uint32_t stride, float* scratch,
                                                  uint32_t* row_tag = nullptr, uint32_t epoch = 0) {
    const uint32_t lane = threadIdx.x;
    {
        const uint32_t groups = a.hidden / 32U, total = a.rows * groups, g0 = qb * 8U;
        float factor = 1.0F;         // (a block's eight groups belong to one row: hidden % 256 == 0)
        if constexpr (NORM) factor = row_norm_factor<KIND>(scratch, a.x + (g0 / groups) * a.x_stride, a.hidden, a.norm_eps);
        for (uint32_t i = 0; i < 8U; i += 2U) {
            const uint32_t g = g0 + i + (lane >> 5), j = lane & 31U;
            if (g < total) {
                const uint32_t r = g / groups, gi = g % groups;
                float v = load_activation<KIND>(a.x + r * a.x_stride, gi * 32U + j);
                if constexpr (NORM) {
                    v = v * factor;
                    if (a.norm_w) v = v * a.norm_w[gi * 32U + j];
                    if (a.normed) a.normed[static_cast<size_t>(r) * a.hidden + gi * 32U + j] = v;
                }
                const float amax = max32(__builtin_fabsf(v));
                const bool tiny = amax > 0.0F && amax < 0x1p-119F;
                const float delta = (amax == 0.0F || tiny) ? 1.0F : amax / 127.0F;
                const int code = a8_code(v, delta, tiny);
                const int sum = sum32_i(code);
                const int bad = or32_i(finite_f(v) ? 0 : 1);
                store_shared_or_plain(LINES, a.codes + static_cast<size_t>(r) * a.hidden + gi * 32U + j, static_cast<int8_t>(code));
                if (j == 0) {
                    store_shared_or_plain(LINES, a.deltas + static_cast<size_t>(r) * groups + gi, delta);
                    store_shared_or_plain(LINES, a.sums + static_cast<size_t>(r) * groups + gi, static_cast<int32_t>(sum));
                    if (bad) atomicOr(&flags[r * stride], static_cast<uint32_t>(MI355_STATUS_NONFINITE_ACTIVATION));
                }
            }
        }
        // the row's last quantiser block publishes the row's status word (a row's 32-groups fill whole blocks: hidden % 256 == 0)
        // (the flag words are read-modify-written by device-scope atomics only; the ticket orders them as above)
        const uint32_t r = g0 / groups;
        if constexpr (LINES) {
            // (the A8 image is written by device-scope stores: waves of the same launch, on other XCDs, read it once the row's tag says so)
            if (arrive_last(&ticket[r * stride], groups / 8U)) {
                if (lane == 0) {
                    __hip_atomic_store(&a.status[r], __hip_atomic_load(&flags[r * stride], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(&flags[r * stride], 0U, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                stores_acknowledged();
                if (lane == 0) __hip_atomic_store(row_tag + r, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        } else {
            __syncthreads();
            if (lane == 0 && __hip_atomic_fetch_add(&ticket[r * stride], 1U, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT) == groups / 8U - 1U) {
                a.status[r] = __hip_atomic_load(&flags[r * stride], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                flags[r * stride] = 0;
                ticket[r * stride] = 0;
            }
        }
    }
}

// Decode router launch (rows <= 16). Blocks [0, route_blocks) run the logit chains of (row, 8 experts). In the plain form
// (a.plan == nullptr) the kernel stops there. In the fused form blocks [route_blocks, route_blocks + quant_blocks)
// quantise the input rows to A8 (8 groups of 32 per block; the last of a row's blocks publishes the row's status word),
// and the block that finishes a row's last 8 experts (row ticket) runs that row's softmax / top-k / weights and writes the
// row's work items: a decode batch is planned one item per assignment (item i = assignment i, order = identity; the CSR
// fields of the plan are not written), so nothing waits for the other rows. Every ticket word is left zero.
template <int KIND, bool NORM = false>
__global__ __launch_bounds__(64) void route_decode_kernel(RouteArgs a) {
    __shared__ ChainSlotT<NORM> slot0;
    __shared__ ChainSlotT<NORM> slot1;
    __shared__ ChainSlotT<NORM> slot2;
    __shared__ ChainSlotT<NORM> slot3;
    __shared__ uint32_t flag;
    ChainSlotT<NORM>* const slots[4] = {&slot0, &slot1, &slot2, &slot3};
    // the scratch of the row's norm factor and of the select lives in the fourth slot, which the ring first fills after the norm
    // factor is known and which is free again once the chain has run: LDS per workgroup stays under half a compute unit's, so a
    // launch of more one-wave workgroups than compute units (16 rows x 160 experts: 320) still runs in one round (61 -> 32 us)
    static_assert(sizeof(ChainSlotT<NORM>) >= kRouteMaxExperts * sizeof(float), "select scratch");
    float* const sel_p = reinterpret_cast<float*>(&slot3);
    const uint32_t bid = blockIdx.x, lane = threadIdx.x, neb = (a.p.experts + 7U) / 8U;
    uint32_t* tickets = a.plan ? a.plan + kPlanTicketsAt : nullptr;
    if (bid < a.route_blocks) {
        const uint32_t row = bid / neb;
        float r = 1.0F;
        if constexpr (NORM) r = row_norm_factor<KIND>(sel_p, a.x + row * a.x_stride, a.hidden, a.norm_eps);
        route_chain_block<KIND, NORM>(slots, a, row, (bid % neb) * 8U, r);
        if (!a.plan) return;
        // hand-off between workgroups: the wave's logit stores happen before the barrier, the barrier before lane 0's
        // ticket increment, which releases them at device scope; the workgroup that takes the row's last ticket acquires with
        // the same operation, and its other lanes read the logits after the second barrier
        __syncthreads();
        if (lane == 0) flag = __hip_atomic_fetch_add(&tickets[row], 1U, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT) == neb - 1U;
        __syncthreads();
        if (flag) {
            if (lane == 0) tickets[row] = 0;
            // The plan of a decode batch. Routed slots: position row * K + slot, one item per assignment. The always-on experts
            // behind them (slot K + s, chosen by every row): positions rows * K + s * rows + row, one item per four rows, so
            // their weights are swept once per four rows and not once per row.
            const uint32_t expert = route_select_row(sel_p, a, row);
            const uint32_t K = a.p.top_k, S = a.p.shared_experts, P = K + S, assignments = a.rows * P, all = a.p.experts + S;
            uint32_t* items = a.plan + plan_items_at(all, assignments);
            uint32_t* order = a.plan + plan_order_at(all);
            if (lane < K) {
                const uint32_t at = row * K + lane;
                *reinterpret_cast<uint4*>(items + 4U * at) = make_uint4(expert, at, at + 1U, row * P + lane + 1U);     // (the item names its assignment)
                order[at] = row * P + lane;
            } else if (lane < P) order[a.rows * K + (lane - K) * a.rows + row] = row * P + lane;
        }
        if (bid == 0) {
            const uint32_t K = a.p.top_k, S = a.p.shared_experts, P = K + S, assignments = a.rows * P, all = a.p.experts + S;
            const uint32_t chunks = (a.rows + 3U) / 4U, made = a.rows * K + S * chunks;
            uint32_t* items = a.plan + plan_items_at(all, assignments);
            if (lane < S * chunks) {
                const uint32_t s_ = lane / chunks, c = lane - s_ * chunks, first = a.rows * K + s_ * a.rows + 4U * c;
                const uint32_t last = 4U * c + 4U < a.rows ? first + 4U : a.rows * K + s_ * a.rows + a.rows;
                *reinterpret_cast<uint4*>(items + 4U * (a.rows * K + lane)) = make_uint4(a.p.experts + s_, first, last, 0U);
            }
            for (uint32_t i = made + lane; i < assignments; i += 64U) *reinterpret_cast<uint4*>(items + 4U * i) = make_uint4(0U, 0U, 0U, 0U);
            if (lane == 0) {
                *a.job_status = 0;
                a.plan[0] = assignments; a.plan[1] = 0; a.plan[2] = S ? 4U : 1U; a.plan[4] = made;
            }
        }
    } else {
        a8_prologue_block<KIND, NORM>(a, bid - a.route_blocks, tickets + 16U, tickets + 128U, 1U, sel_p);
    }
}

// softmax / top-k / weights, one row per one-wave block (the plain router).
__global__ __launch_bounds__(64) void route_select_kernel(RouteArgs a) {
    __shared__ __attribute__((aligned(16))) float sel_p[kRouteMaxExperts];
    route_select_row(sel_p, a, blockIdx.x);
}

// ======================================================================================================== expert plan
// (layout of the plan words: see the router section above)

// The routes of a batch as the plan kernels read them: assignment a = row a / top_k, slot a % top_k, rows `rs` bytes apart.
struct RoutesView {
    const uint32_t* base;
    uint64_t rs;
    uint32_t top_k;
    __device__ __forceinline__ uint32_t at(uint32_t a) const {
        if (rs == 4ULL * top_k) return base[a];
        const uint32_t row = a / top_k;
        return reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint8_t*>(base) + row * rs)[a - row * top_k];
    }
};
inline RoutesView dense_routes(const uint32_t* routes, uint32_t top_k) { return RoutesView{routes, 4ULL * top_k, top_k}; }

// Stable order of a large batch: one 16-wave workgroup per expert. Every wave owns a contiguous sixteenth of the assignments:
// it first counts its own assignments of the expert (ballot + population count, 64 at a time), the counts of the waves before
// it give its first position, and a second walk places them in index order (the offsets are already in the plan).
__global__ __launch_bounds__(1024) void plan_order_kernel(RoutesView routes, uint32_t experts, uint32_t assignments, uint32_t* plan) {
    __shared__ uint32_t wave_count[16];
    const uint32_t e = blockIdx.x, lane = threadIdx.x & 63U, wave = threadIdx.x >> 6;
    const uint32_t first = plan[kPlanOffsetsAt + e], end = plan[kPlanOffsetsAt + e + 1];
    if (first == end) return;                                   // uniform over the workgroup
    const uint32_t per = ((assignments + 15U) / 16U + 63U) & ~63U;
    const uint32_t lo = wave * per < assignments ? wave * per : assignments, hi = lo + per < assignments ? lo + per : assignments;
    uint32_t mine_total = 0;
    for (uint32_t a0 = lo; a0 < hi; a0 += 64U) {
        const uint32_t a = a0 + lane;
        mine_total += static_cast<uint32_t>(__popcll(__ballot(a < hi && routes.at(a) == e)));
    }
    if (lane == 0) wave_count[wave] = mine_total;
    __syncthreads();
    uint32_t at = first;
    for (uint32_t w = 0; w < wave; ++w) at += wave_count[w];
    const uint32_t stop = at + mine_total;
    uint32_t* order = plan + plan_order_at(experts);
    for (uint32_t a0 = lo; a0 < hi && at < stop; a0 += 64U) {
        const uint32_t a = a0 + lane;
        const bool mine = a < hi && routes.at(a) == e;
        const uint64_t votes = __ballot(mine);
        if (mine) order[at + __popcll(votes & ((1ULL << lane) - 1ULL))] = a;
        at += static_cast<uint32_t>(__popcll(votes));
    }
}

// Exclusive prefix sum of one value per thread over a 1024-thread workgroup (16 waves); `total` is the sum over all threads.
// wave_totals: 16 shared words of the caller's, not reused before its next barrier.
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t v, uint32_t* wave_totals, uint32_t& total) {
    const uint32_t lane = threadIdx.x & 63U, wave = threadIdx.x >> 6;
    uint32_t x = v;
#pragma unroll
    for (uint32_t d = 1; d < 64U; d <<= 1) {
        const uint32_t below = __shfl_up(x, d);
        if (lane >= d) x += below;
    }
    if (lane == 63U) wave_totals[wave] = x;
    __syncthreads();
    uint32_t base = 0, sum = 0;
    for (uint32_t w = 0; w < 16U; ++w) {
        const uint32_t t = wave_totals[w];
        base += w < wave ? t : 0U;
        sum += t;
    }
    total = sum;
    return base + x - v;
}

// The expert plan in one workgroup: thread e owns expert e (counts by shared-memory atomics, three prefix sums for the
// offsets, the item numbers and the touched list, then its own items and - for a small batch - its own stretch of the order).
__global__ __launch_bounds__(1024) void plan_kernel(RoutesView routes, uint32_t experts, uint32_t assignments, uint32_t split,
                                                    uint32_t item_bound, uint32_t fill_order, uint32_t* plan) {
    __shared__ uint32_t count[kRouteMaxExperts];
    __shared__ uint32_t wave_totals[3][16];
    __shared__ uint32_t wave_largest[16];
    __shared__ uint32_t small_routes[256];                 // fill_order: at most 256 assignments
    const uint32_t tid = threadIdx.x, lane = tid & 63U, wave = tid >> 6;
    count[tid] = 0;
    __syncthreads();
    for (uint32_t a = tid; a < assignments; a += 1024U) {
        const uint32_t e = routes.at(a);
        if (fill_order) small_routes[a] = e;
        if (e < experts) atomicAdd(&count[e], 1U);
    }
    __syncthreads();
    const uint32_t c = tid < experts ? count[tid] : 0U, pieces = (c + split - 1U) / split;
    uint32_t run, made, touched;
    const uint32_t first = block_exclusive_scan(c, wave_totals[0], run);
    const uint32_t item_from = block_exclusive_scan(pieces, wave_totals[1], made);
    const uint32_t touched_from = block_exclusive_scan(c != 0 ? 1U : 0U, wave_totals[2], touched);
    uint32_t largest = c;
#pragma unroll
    for (int d = 32; d; d >>= 1) {
        const uint32_t other = __shfl_xor(largest, d);
        largest = other > largest ? other : largest;
    }
    if (lane == 0) wave_largest[wave] = largest;
    __syncthreads();
    uint32_t* offsets = plan + kPlanOffsetsAt;
    uint32_t* touched_ids = plan + plan_touched_at(experts);
    uint32_t* order = plan + plan_order_at(experts);
    uint32_t* items = plan + plan_items_at(experts, assignments);
    if (tid < experts) {
        offsets[tid] = first;
        if (c != 0) {
            touched_ids[touched_from] = tid;
            for (uint32_t b = 0, k = item_from; b < c; b += split, ++k)
                *reinterpret_cast<uint4*>(items + 4U * k) = make_uint4(tid, first + b, first + (b + split < c ? b + split : c), 0U);
        }
    }
    for (uint32_t u = made + tid; u < item_bound; u += 1024U) *reinterpret_cast<uint4*>(items + 4U * u) = make_uint4(0U, 0U, 0U, 0U);
    if (tid == 0) {
        uint32_t most = 0;
        for (uint32_t w = 0; w < 16U; ++w) most = wave_largest[w] > most ? wave_largest[w] : most;
        offsets[experts] = run;
        plan[0] = assignments; plan[1] = touched; plan[2] = most; plan[4] = made;
    }
    if (!fill_order || tid >= experts || c == 0) return;   // large batches: plan_order_kernel follows
    uint32_t at = first;
    for (uint32_t a = 0; a < assignments; ++a)
        if (small_routes[a] == tid) order[at++] = a;
}

__global__ __launch_bounds__(64) void clear_validate_kernel(const uint32_t* routes, const float* route_weights, uint32_t experts,
                                                            uint32_t top_k, uint32_t* status, uint32_t* job_status) {
    const uint32_t row = blockIdx.x;
    uint32_t bad = 0;
    for (uint32_t k = threadIdx.x; k < top_k; k += 64U) {
        if (routes[row * top_k + k] >= experts) bad = MI355_STATUS_INVALID_ROUTE;
        if (route_weights && !finite_f(route_weights[row * top_k + k])) bad = MI355_STATUS_INVALID_ROUTE;
    }
    for (int d = 32; d; d >>= 1) bad |= __shfl_xor(bad, d);
    if (threadIdx.x == 0) {
        status[row] = bad;
        if (row == 0) *job_status = 0;
    }
}

// ======================================================================================================== Q4_K x A8 rows
// gate + up + SwiGLU + A8 re-quantisation: one wavefront per (touched expert, 32-output group). Lanes 0..31 hold the
// gate rows of the group, lanes 32..63 the up rows; one cross-half exchange pairs them, then both halves evaluate the
// same 32-value h group.
// Reference: src/cpu/core/routed_expert.cpp:403-427 (gate item), :147-170 (swiglu_quantize).
template <int NA, class IndexOf>
__device__ __forceinline__ void project_epilogue(const float (&value)[NA], const mi355_moe_weights& w, const RowsK& r, uint32_t grp, IndexOf index_of);

// index_of(a): the assignment index of the sweep's activation row a < NA (a may differ between lanes).
template <int NA, int DEPTH, bool NARROW = false, class IndexOf>
__device__ __forceinline__ void project_chunk_of(lds_u8* const (&slots)[DEPTH], const StageSource& source, const mi355_moe_weights& w,
                                                 const RowsK& r, uint32_t grp, IndexOf index_of) {
    const uint32_t lane = threadIdx.x & 63U, o = lane & 31U;
    uint32_t sidx[NA], src[NA], lane_rows[(NA + 3) / 4];
#pragma unroll
    for (int a = 0; a < NA; ++a) {
        sidx[a] = __builtin_amdgcn_readfirstlane(index_of(static_cast<uint32_t>(a)));
        src[a] = r.row_of(sidx[a]);
    }
#pragma unroll
    for (int h = 0; h < (NA + 3) / 4; ++h) {
        const uint32_t a = 4U * h + (lane >> 4);
        lane_rows[h] = r.row_of(index_of(a < static_cast<uint32_t>(NA) ? a : 0U));
    }
    const ActRows<NA> act(r.in, src, lane_rows);
    float value[NA];
    sweep_rows<NA, DEPTH, NARROW>(slots, source, w.hidden / 256U, act, value);
    project_epilogue<NA>(value, w, r, grp, index_of);
}

// SwiGLU + A8 re-quantisation of one 32-output group: lanes 0..31 hold the gate values, lanes 32..63 the up values of outputs
// 32 grp .. 32 grp + 31 for each of the NA assignments index_of(0 .. NA - 1). Reference: src/cpu/core/routed_expert.cpp:147-170.
template <int NA, class IndexOf>
__device__ __forceinline__ void project_epilogue(const float (&value)[NA], const mi355_moe_weights& w, const RowsK& r, uint32_t grp, IndexOf index_of) {
    const uint32_t lane = threadIdx.x & 63U, o = lane & 31U;
    uint32_t sidx[NA], src[NA];
#pragma unroll
    for (int a = 0; a < NA; ++a) {
        sidx[a] = __builtin_amdgcn_readfirstlane(index_of(static_cast<uint32_t>(a)));
        src[a] = r.row_of(sidx[a]);
    }
    const bool ds = r.awords != nullptr;      // early routes: device-scope stores (an assignment may be written again by a repair)
#pragma unroll
    for (int a = 0; a < NA; ++a) {
        const float other = __shfl_xor(value[a], 32);
        const float g = lane < 32U ? value[a] : other, u = lane < 32U ? other : value[a];
        float gc = g, uc = u;
        swiglu_clamp(gc, uc, w.swiglu_limit);
        const float h = (gc / (1.0F + exp_of(w.exp_kind, -gc))) * uc;
        const uint32_t at_out = grp * 32U + o;
        if (lane < 32U) {
            if (r.gate_out) store_shared_or_plain(ds, r.inter_of(r.gate_out, sidx[a]) + at_out, g);
            if (r.up_out) store_shared_or_plain(ds, r.inter_of(r.up_out, sidx[a]) + at_out, u);
            if (r.h_out) store_shared_or_plain(ds, r.inter_of(r.h_out, sidx[a]) + at_out, h);
        }
        if (!r.h.codes) continue;                         // projection only (the probe form): no A8 image of h
        if (or32_i((finite_f(g) && finite_f(u) && finite_f(h)) ? 0 : 1)) {
            if (lane == 0) {
                if (r.awords) atomicOr(&r.awords[sidx[a]], 0x80000000U);        // early routes: per assignment, folded by the down launch
                else {
                    atomicOr(r.status_of(src[a]), r.nonfinite_bit);
                    atomicOr(r.job_status, static_cast<uint32_t>(MI355_STATUS_NONFINITE_PROJECTION));
                }
            }
        } else {
            const float amax = max32(__builtin_fabsf(h));
            const bool tiny = amax > 0.0F && amax < 0x1p-119F;
            const float dl = (amax == 0.0F || tiny) ? 1.0F : amax / 127.0F;
            const int code = a8_code(h, dl, tiny);
            const int sum = sum32_i(code);
            if (lane < 32U) store_shared_or_plain(ds, r.h_codes_of(sidx[a]) + at_out, static_cast<int8_t>(code));
            if (lane == 0) {
                store_shared_or_plain(ds, r.h_deltas_of(sidx[a]) + grp, dl);
                store_shared_or_plain(ds, r.h_sums_of(sidx[a]) + grp, static_cast<int32_t>(sum));
            }
        }
    }
}

template <int NA, int DEPTH, bool NARROW = false>
__device__ __forceinline__ void project_chunk(lds_u8* const (&slots)[DEPTH], const StageSource& source, const mi355_moe_weights& w,
                                              const RowsK& r, uint32_t grp, uint32_t order_at, uint32_t c0) {
    project_chunk_of<NA, DEPTH, NARROW>(slots, source, w, r, grp, [&](uint32_t a) { return ordered(r, order_at, c0 + a); });
}

#define STRIX_RING_SLOTS(DEPTH, NBMAX)                                                           \
    __shared__ __attribute__((aligned(16))) uint8_t ring0[slot_bytes(NBMAX)];                    \
    __shared__ __attribute__((aligned(16))) uint8_t ring1[slot_bytes(NBMAX)];                    \
    __shared__ __attribute__((aligned(16))) uint8_t ring2[DEPTH > 2 ? slot_bytes(NBMAX) : 16];   \
    __shared__ __attribute__((aligned(16))) uint8_t ring3[DEPTH > 3 ? slot_bytes(NBMAX) : 16];   \
    lds_u8* const ring[4] = {(lds_u8*)ring0, (lds_u8*)ring1, (lds_u8*)ring2, (lds_u8*)ring3};    \
    lds_u8* slots[DEPTH];                                                                        \
    _Pragma("unroll") for (int i = 0; i < DEPTH; ++i) slots[i] = ring[i];

// NBMAX = most activation rows sharing one sweep of the weights (4 for routed experts, 8 for a dense matrix).
template <int NBMAX, int DEPTH>
__global__ __launch_bounds__(64, DEPTH > 3 ? 1 : 2) void project_wave_kernel(mi355_moe_weights w, RowsK r, uint32_t assignments) {
    STRIX_RING_SLOTS(DEPTH, NBMAX)
    const WorkItem item = work_item(w, r, plan_items_at(w.experts, assignments), blockIdx.y);
    const uint32_t e = __builtin_amdgcn_readfirstlane(item.e), begin = __builtin_amdgcn_readfirstlane(item.begin), end = __builtin_amdgcn_readfirstlane(item.end);
    if (begin == end) return;
    // a wave that serves several activation rows has the longest instruction stream of the launch: let it issue first
    if (end - begin > 1U) __builtin_amdgcn_s_setprio(3);
    const uint32_t order_at = plan_order_at(w.experts);
    const uint32_t grp = blockIdx.x;
    const size_t base = static_cast<size_t>(e) * w.gate_expert_stride + static_cast<size_t>(grp * 32U) * w.gate_row_stride;
    const uint8_t* gate = w.gate + base;
    const uint8_t* up = w.up + base;
    const size_t stride = w.gate_row_stride;       // (64-bit: row * stride passes 2^32 for rows of 64 MiB and more)
    StageSource source;
    source.init([&](uint32_t row) { return row < 32U ? gate + row * stride : up + (row - 32U) * stride; });
    lds_u8* const (&sl)[DEPTH] = slots;
    for (uint32_t c0 = begin; c0 < end;) {
        const uint32_t left = end - c0, na = left < static_cast<uint32_t>(NBMAX) ? left : static_cast<uint32_t>(NBMAX);
        switch (na) {
        case 1: project_chunk<1, DEPTH>(sl, source, w, r, grp, order_at, c0); break;
        case 2: project_chunk<2, DEPTH>(sl, source, w, r, grp, order_at, c0); break;
        case 3: project_chunk<3, DEPTH>(sl, source, w, r, grp, order_at, c0); break;
        case 4: project_chunk<4, DEPTH>(sl, source, w, r, grp, order_at, c0); break;
        default:
            if constexpr (NBMAX == 8) {
                switch (na) {
                case 5: project_chunk<5, DEPTH>(sl, source, w, r, grp, order_at, c0); break;
                case 6: project_chunk<6, DEPTH>(sl, source, w, r, grp, order_at, c0); break;
                case 7: project_chunk<7, DEPTH>(sl, source, w, r, grp, order_at, c0); break;
                default: project_chunk<8, DEPTH>(sl, source, w, r, grp, order_at, c0); break;
                }
            }
            break;
        }
        c0 += na;
    }
}

// ---- the front launch of a decode batch planned from early routes (route_early.hpp) ----------------------------------
// One-wave workgroups, in dispatch order:
//   early blocks (row, 4 experts): lane-parallel logits; the block that completes a row picks the row's experts, clears the
//     row's assignment words and publishes one tag {epoch, expert} per assignment;
//   A8 prologue blocks: the A8 image of the input rows; the block that completes a row publishes the row's status word and tag;
//   side blocks (row, 2 experts): the exact logit chains; the block that completes a row runs the exact softmax / top-k / weights
//     (the caller's ids, weights and scores), writes the row's work items (the exact experts: what the down launch reads) and
//     compares its ids with the early ones: where they differ it waits until the assignment's speculative waves have all
//     finished (their count in the assignment's word), clears the word's non-finite flag and recomputes the assignment's h image
//     on the exact expert;
//   projection blocks (assignment, 32-output group): wait for the assignment's tag and the row's tag, then one sweep of the
//     tagged expert's gate / up rows; each counts itself into its assignment's word when its part of the h image is acknowledged.
// Blocks are dispatched in index order, so what a waiting block waits for has been dispatched before it (the repair waits for
// projection blocks, which themselves wait only for blocks in front of them); every wait is bounded, and a wait that runs out (it
// cannot, short of a lost launch) flags the row as an invalid route: nothing of it is published. Everything that crosses
// workgroups inside the launch - logits, tags, counts, the A8 images of x and of h, the optional fp32 intermediates - moves by
// device-scope stores and loads (an assignment that is repaired is written twice, by waves of different XCDs, and the later
// write has to win at the memory side).
// A waiting wave polls rarely at first and sleeps between polls: a thousand waves polling one line at full rate saturate the
// L2 channel that holds it, and every weight stream crossing that channel with it.
// Two ring slots of 10,240 bytes: eight workgroups share a compute unit.
constexpr uint32_t kFrontSpinLimit = 1U << 22;
struct FrontBlocks { uint32_t early, prologue, side; };

// gate + up + SwiGLU + A8 of assignment `at` on expert e, outputs 32 grp .. 32 grp + 31: rows in dense GGUF order stream as
// contiguous stages (q4k_blocks.hpp), others as one super-block of each row per stage.
__device__ __forceinline__ void front_project(lds_u8* const (&slots)[2], const mi355_moe_weights& w, const RowsK& r, uint32_t e, uint32_t grp, uint32_t at) {
    const size_t base = static_cast<size_t>(e) * w.gate_expert_stride + static_cast<size_t>(grp * 32U) * w.gate_row_stride;
    const uint8_t* gate = w.gate + base;
    const uint8_t* up = w.up + base;
    const uint32_t B = w.hidden / 256U;
    if (w.gate_row_stride == static_cast<uint64_t>(B) * kQ4kBlock && block_lanes_ok(B, 32U)) {
        const BlockLanes g = block_lanes(B, 32U);
        const uint32_t half = 32U / g.R;                  // stages of the gate rows, then as many of the up rows
        float value[1];
        const auto stage_base = [&](uint32_t s) { return s < half ? gate + static_cast<size_t>(s) * g.stage_bytes : up + static_cast<size_t>(s - half) * g.stage_bytes; };
        if (g.used == 64U && half == 4U) value[0] = sweep_block_lanes_terms<8>(slots, stage_base, g, r.in, r.row_of(at));      // (hidden 2048)
        else if (g.used == 64U && half == 2U) value[0] = sweep_block_lanes_terms<4>(slots, stage_base, g, r.in, r.row_of(at)); // (hidden 1024)
        else value[0] = sweep_block_lanes<2>(slots, stage_base, 2U * half, g, r.in, r.row_of(at));
        project_epilogue<1>(value, w, r, grp, [&](uint32_t) { return at; });
        return;
    }
    const size_t stride = w.gate_row_stride;
    StageSource source;
    source.init([&](uint32_t q) { return q < 32U ? gate + q * stride : up + (q - 32U) * stride; });
    project_chunk<1, 2>(slots, source, w, r, grp, 0U, at);
}

template <int KIND>
__device__ __forceinline__ void side_router_block(lds_u8* const (&slots)[2], const mi355_moe_weights& w, const RowsK& r,
                                                  const RouteArgs& a, uint32_t sb, uint32_t assignments, uint32_t epoch) {
    const uint32_t lane = threadIdx.x & 63U, neb = (a.p.experts + kSideExperts - 1U) / kSideExperts, row = sb / neb;
    side_chain_block<KIND>(slots[0], slots[1], a, row, (sb % neb) * kSideExperts);
    uint32_t* lines = a.plan + kPlanLinesAt;
    if (!arrive_last(&lines[kLinesSide + row * kLineWords], neb)) return;
    const uint32_t expert = route_select_row(reinterpret_cast<float*>((uint8_t*)slots[0]), a, row);
    const uint32_t K = a.p.top_k, groups = w.ffn / 32U;
    if (lane < K) {
        const uint32_t at = row * K + lane;
        *reinterpret_cast<uint4*>(a.plan + plan_items_at(w.experts, assignments) + 4U * at) = make_uint4(expert, at, at + 1U, at + 1U);
        a.plan[plan_order_at(w.experts) + at] = at;
    }
    // the early choice of this row and the A8 image of its input (the repair reads it)
    const unsigned long long* etags = reinterpret_cast<const unsigned long long*>(a.plan + kPlanEtagsAt);
    unsigned long long tag = 0;
    uint32_t image = 0;
    bool there = false;
    for (uint32_t spins = 0; spins < kFrontSpinLimit && !there; ++spins) {
        if (lane < K) tag = __hip_atomic_load(&etags[row * K + lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        image = __hip_atomic_load(&lines[kLinesRowTags + row], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        there = __ballot(lane < K && static_cast<uint32_t>(tag >> 32) != epoch) == 0 && image == epoch;
        if (!there) __builtin_amdgcn_s_sleep(16);
    }
    asm volatile("" ::: "memory");
    if (!there) {
        if (lane == 0) atomicOr(r.status_of(row), static_cast<uint32_t>(MI355_STATUS_INVALID_ROUTE));
        return;
    }
    uint64_t differ = __ballot(lane < K && static_cast<uint32_t>(tag) != expert);
    // Most differences are the same experts in another order (two scores closer than the early logits resolve): the h image
    // such a slot needs exists already, under the slot that held its expert, and is copied. Only an expert the early choice did not
    // hold at all is swept again. (With the optional fp32 intermediates bound every differing slot is swept again.)
    const uint32_t image_words = w.ffn / 4U + 2U * groups;         // codes, deltas, sums of one assignment, in 32-bit words
    if (differ && !r.gate_out && !r.up_out && !r.h_out && K * image_words * 4U <= kSideSlotBytes) {
        uint32_t src = 0xffU;
        for (uint32_t j = 0; j < K; ++j) {
            const uint32_t held = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(tag)), static_cast<int>(j)));
            if (lane < K && expert == held) src = j;
        }
        uint64_t copy = __ballot(lane < K && ((differ >> lane) & 1ULL) && src != 0xffU);
        if (copy) {
            // every speculative wave of the row has to be through: a slot is read as a source or overwritten as a destination
            bool through = false;
            for (uint32_t spins = 0; spins < kFrontSpinLimit && !through; ++spins) {
                const uint32_t seen = lane < K ? __hip_atomic_load(&r.awords[row * K + lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & 0xffffU : groups;
                through = __ballot(seen < groups) == 0;
                if (!through) __builtin_amdgcn_s_sleep(32);
            }
            asm volatile("" ::: "memory");
            if (!through) {
                if (lane == 0) atomicOr(r.status_of(row), static_cast<uint32_t>(MI355_STATUS_INVALID_ROUTE));
                return;
            }
            const auto image_word = [&](uint32_t at, uint32_t i) -> uint32_t* {
                if (i < w.ffn / 4U) return reinterpret_cast<uint32_t*>(r.h_codes_of(at)) + i;
                if (i < w.ffn / 4U + groups) return reinterpret_cast<uint32_t*>(r.h_deltas_of(at)) + (i - w.ffn / 4U);
                return reinterpret_cast<uint32_t*>(r.h_sums_of(at)) + (i - w.ffn / 4U - groups);
            };
            uint32_t* stage = reinterpret_cast<uint32_t*>((uint8_t*)slots[0]);
            uint32_t flags = 0;                                   // bit k: the source of slot k carried the non-finite flag
            for (uint64_t left = copy; left;) {                   // all sources first: a source may itself be a destination
                const uint32_t k = static_cast<uint32_t>(__ffsll(static_cast<long long>(left))) - 1U;
                left &= left - 1ULL;
                const uint32_t from = row * K + static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(src), static_cast<int>(k)));
                for (uint32_t i = lane; i < image_words; i += 64U) stage[k * image_words + i] = __hip_atomic_load(image_word(from, i), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                flags |= (__hip_atomic_load(&r.awords[from], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >> 31) << k;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            for (uint64_t left = copy; left;) {
                const uint32_t k = static_cast<uint32_t>(__ffsll(static_cast<long long>(left))) - 1U;
                left &= left - 1ULL;
                const uint32_t to = row * K + k;
                for (uint32_t i = lane; i < image_words; i += 64U) __hip_atomic_store(image_word(to, i), stage[k * image_words + i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (lane == 0) __hip_atomic_store(&r.awords[to], groups | (((flags >> k) & 1U) << 31), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");      // the staged images are out of LDS before a sweep reuses the slot
            differ &= ~copy;
        }
    }
    while (differ) {
        const uint32_t k = static_cast<uint32_t>(__ffsll(static_cast<long long>(differ))) - 1U;
        differ &= differ - 1ULL;
        const uint32_t at = row * K + k, e = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(expert), static_cast<int>(k)));
        uint32_t seen = 0;
        for (uint32_t spins = 0; spins < kFrontSpinLimit; ++spins) {
            seen = __hip_atomic_load(&r.awords[at], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & 0xffffU;
            if (seen >= groups) break;
            __builtin_amdgcn_s_sleep(32);
        }
        asm volatile("" ::: "memory");
        if (seen < groups) {
            if (lane == 0) atomicOr(r.status_of(row), static_cast<uint32_t>(MI355_STATUS_INVALID_ROUTE));
            continue;
        }
        if (lane == 0) __hip_atomic_store(&r.awords[at], groups, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (uint32_t grp = 0; grp < groups; ++grp) front_project(slots, w, r, e, grp, at);
    }
}

template <int KIND>
__global__ __launch_bounds__(64, 2) void layer_front_kernel(mi355_moe_weights w, RowsK r, uint32_t assignments, RouteArgs a, FrontBlocks nb) {
    // exactly 20,480 bytes of LDS: eight workgroups fill a compute unit's 160 KB (one more byte and only seven fit)
    __shared__ __attribute__((aligned(16))) uint8_t ring0[kSideSlotBytes];
    __shared__ __attribute__((aligned(16))) uint8_t ring1[kSideSlotBytes];
    static_assert(kSideSlotBytes == slot_bytes(4), "the projection sweep's slot");
    lds_u8* const slots[2] = {(lds_u8*)ring0, (lds_u8*)ring1};
    lds_u8* const (&sl)[2] = slots;
    uint32_t bid = blockIdx.x;
    const uint32_t lane = threadIdx.x, K = a.p.top_k;
    uint32_t* lines = a.plan + kPlanLinesAt;
    const uint32_t epoch = lines[kLinesEpoch] + 1U;                 // (stored back by the down launch of this call)
    unsigned long long* etags = reinterpret_cast<unsigned long long*>(a.plan + kPlanEtagsAt);
    if (bid < nb.early) {
        const uint32_t neb = (a.p.experts + kEarlyExperts - 1U) / kEarlyExperts, row = bid / neb;
        // the row's first early block also selects: it clears the row's assignment words before anything else (acknowledged long before
        // its tags go out), brings its own four logits, then reads the row's logits until every one carries this call's epoch
        const bool selects = bid % neb == 0;
        if (selects && lane < K) __hip_atomic_store(&r.awords[row * K + lane], 0U, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        early_logits_block<KIND>(a, row, (bid % neb) * kEarlyExperts, epoch);
        if (bid == 0 && lane == 0) {
            *a.job_status = 0;
            a.plan[0] = assignments; a.plan[1] = 0; a.plan[2] = 1U; a.plan[4] = assignments;
        }
        if (!selects) return;
        bool ok;
        const uint32_t expert = early_select_row(a, row, epoch, ok);
        if (!ok) {
            if (lane == 0) atomicOr(r.status_of(row), static_cast<uint32_t>(MI355_STATUS_INVALID_ROUTE));
            return;
        }
        stores_acknowledged();
        if (lane < K) __hip_atomic_store(&etags[row * K + lane], (static_cast<unsigned long long>(epoch) << 32) | expert, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return;
    }
    bid -= nb.early;
    if (bid < nb.prologue) {
        a8_prologue_block<KIND, false, true>(a, bid, lines + kLinesPrologue, lines + kLinesPrologue + 1U, kLineWords, nullptr, lines + kLinesRowTags, epoch);
        return;
    }
    bid -= nb.prologue;
    if (bid < nb.side) {
        side_router_block<KIND>(sl, w, r, a, bid, assignments, epoch);
        return;
    }
    bid -= nb.side;
    // Projection block: assignment `at`, 32-output group `grp`. (Sharing one sweep among the rows that chose an expert was
    // measured slower: the sweeps that serve several rows finish last, and the others do not speed up.)
    const uint32_t groups = w.ffn / 32U, at = bid / groups, grp = bid - at * groups, row = at / K;
    unsigned long long tag = 0;
    uint32_t image = 0;
    bool there = false;
    for (uint32_t spins = 0; spins < kFrontSpinLimit && !there; ++spins) {
        tag = __hip_atomic_load(&etags[at], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        image = __hip_atomic_load(&lines[kLinesRowTags + row], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        there = static_cast<uint32_t>(tag >> 32) == epoch && image == epoch;
        // a block that finds nothing at its first look started with the launch: the tags are microseconds away (one long sleep,
        // about 3 us); a block dispatched later, into a freed slot, finds them at once
        if (!there) { if (spins == 0) __builtin_amdgcn_s_sleep(127); else __builtin_amdgcn_s_sleep(8); }
    }
    asm volatile("" ::: "memory");
    if (!there) {
        if (lane == 0) atomicOr(r.status_of(row), static_cast<uint32_t>(MI355_STATUS_INVALID_ROUTE));
        return;
    }
    const uint32_t e = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(static_cast<uint32_t>(tag))));
    // The compute unit issues its oldest waves first, so the blocks dispatched last fall behind the others stage by stage and the
    // launch ends with a few hundred of them alone on the memory system: the later a block's place in the dispatch, the higher
    // its issue priority (the launch at 8 rows: 0.3 - 0.5 us).
    {
        const uint32_t quarter = bid * 4U / (assignments * groups);
        if (quarter == 1U) __builtin_amdgcn_s_setprio(1);
        else if (quarter == 2U) __builtin_amdgcn_s_setprio(2);
        else if (quarter == 3U) __builtin_amdgcn_s_setprio(3);
    }
    front_project(sl, w, r, e, grp, at);
    stores_acknowledged();
    if (lane == 0) __hip_atomic_fetch_add(&r.awords[at], 1U, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// down rows: one wavefront per (touched expert, 64 hidden outputs), lane = output row.
// Reference: src/cpu/core/routed_expert.cpp:429-447 (down item), src/moe_a8_down_contract.cpp:146 (Q4_K down row).
template <int NA, int DEPTH>
__device__ __forceinline__ void down_chunk(lds_u8* const (&slots)[DEPTH], const StageSource& source, const mi355_moe_weights& w,
                                           const RowsK& r, uint32_t order_at, uint32_t c0) {
    uint32_t src[NA], lane_rows[(NA + 3) / 4];
#pragma unroll
    for (int a = 0; a < NA; ++a) src[a] = __builtin_amdgcn_readfirstlane(ordered(r, order_at, c0 + a));
#pragma unroll
    for (int h = 0; h < (NA + 3) / 4; ++h) {
        const uint32_t a = 4U * h + ((threadIdx.x & 63U) >> 4);
        lane_rows[h] = ordered(r, order_at, c0 + (a < static_cast<uint32_t>(NA) ? a : 0U));
    }
    const ActRows<NA> act(r.h, src, lane_rows);
    float value[NA];
    sweep_rows<NA, DEPTH>(slots, source, w.ffn / 256U, act, value);
    const uint32_t o = blockIdx.x * 64U + (threadIdx.x & 63U);
#pragma unroll
    for (int a = 0; a < NA; ++a) r.rawdots_of(src[a], w.hidden)[o] = value[a];
}

template <int NBMAX, int DEPTH>
__global__ __launch_bounds__(64, DEPTH > 3 ? 1 : 2) void down_wave_kernel(mi355_moe_weights w, RowsK r, uint32_t assignments) {
    STRIX_RING_SLOTS(DEPTH, NBMAX)
    const WorkItem item = work_item(w, r, plan_items_at(w.experts, assignments), blockIdx.y);
    const uint32_t e = __builtin_amdgcn_readfirstlane(item.e), begin = __builtin_amdgcn_readfirstlane(item.begin), end = __builtin_amdgcn_readfirstlane(item.end);
    if (begin == end) return;
    if (*r.job_status & MI355_STATUS_NONFINITE_PROJECTION) return;
    if (end - begin > 1U) __builtin_amdgcn_s_setprio(3);     // as in the projection: the longest instruction streams issue first
    const uint32_t order_at = plan_order_at(w.experts);
    const uint8_t* rows = w.down + static_cast<size_t>(e) * w.down_expert_stride + static_cast<size_t>(blockIdx.x * 64U) * w.down_row_stride;
    const size_t stride = w.down_row_stride;
    StageSource source;
    source.init([&](uint32_t row) { return rows + row * stride; });
    lds_u8* const (&sl)[DEPTH] = slots;
    for (uint32_t c0 = begin; c0 < end;) {
        const uint32_t left = end - c0, na = left < static_cast<uint32_t>(NBMAX) ? left : static_cast<uint32_t>(NBMAX);
        switch (na) {
        case 1: down_chunk<1, DEPTH>(sl, source, w, r, order_at, c0); break;
        case 2: down_chunk<2, DEPTH>(sl, source, w, r, order_at, c0); break;
        case 3: down_chunk<3, DEPTH>(sl, source, w, r, order_at, c0); break;
        case 4: down_chunk<4, DEPTH>(sl, source, w, r, order_at, c0); break;
        default:
            if constexpr (NBMAX == 8) {
                switch (na) {
                case 5: down_chunk<5, DEPTH>(sl, source, w, r, order_at, c0); break;
                case 6: down_chunk<6, DEPTH>(sl, source, w, r, order_at, c0); break;
                case 7: down_chunk<7, DEPTH>(sl, source, w, r, order_at, c0); break;
                default: down_chunk<8, DEPTH>(sl, source, w, r, order_at, c0); break;
                }
            }
            break;
        }
        c0 += na;
    }
}

#include "q4k_mma_moe.hpp"

// ---- the smallest decode batches: 16 rows per wavefront, lane = (row, pair) (q4k_quads.hpp) ------------------------------
#define STRIX_QUAD_SLOTS(DEPTH)                                                                      \
    __shared__ __attribute__((aligned(16))) uint8_t quad0[4][kQuadSlotBytes];                         \
    __shared__ __attribute__((aligned(16))) uint8_t quad1[4][kQuadSlotBytes];                         \
    __shared__ __attribute__((aligned(16))) uint8_t quad2[DEPTH > 2 ? 4 : 1][DEPTH > 2 ? kQuadSlotBytes : 16]; \
    __shared__ __attribute__((aligned(16))) uint8_t quad3[DEPTH > 3 ? 4 : 1][DEPTH > 3 ? kQuadSlotBytes : 16]; \
    const uint32_t wave = threadIdx.x >> 6;                                                           \
    lds_u8* const quad_ring[4] = {(lds_u8*)quad0[wave], (lds_u8*)quad1[wave], (lds_u8*)quad2[DEPTH > 2 ? wave : 0], (lds_u8*)quad3[DEPTH > 3 ? wave : 0]}; \
    lds_u8* slots[DEPTH];                                                                             \
    _Pragma("unroll") for (int i = 0; i < DEPTH; ++i) slots[i] = quad_ring[i];

// gate + up + SwiGLU + A8 of one item (one assignment): a 4-wave workgroup per 32-output group, wave = 8 gate rows and the
// 8 up rows of the same features. Reference: src/cpu/core/routed_expert.cpp:403-427, :147-170.
template <int DEPTH>
__global__ __launch_bounds__(256) void project_quad_kernel(mi355_moe_weights w, RowsK r, uint32_t assignments) {
    STRIX_QUAD_SLOTS(DEPTH)
    __shared__ float wg_amax[4];
    __shared__ int wg_sum[4], wg_bad[4];
    const WorkItem item = work_item(w, r, plan_items_at(w.experts, assignments), blockIdx.y);
    const uint32_t e = item.e, begin = item.begin, end = item.end;
    if (begin == end) return;
    const uint32_t lane = threadIdx.x & 63U, p = lane & 3U, rr = lane >> 2, grp = blockIdx.x;
    const uint32_t sidx = __builtin_amdgcn_readfirstlane(ordered(r, plan_order_at(w.experts), begin)), row = r.row_of(sidx);
    const uint32_t f0 = grp * 32U + 8U * wave;
    const size_t base = static_cast<size_t>(e) * w.gate_expert_stride + static_cast<size_t>(f0) * w.gate_row_stride;
    const uint8_t* gate = w.gate + base;
    const uint8_t* up = w.up + base;
    const size_t stride = w.gate_row_stride;
    QuadSource source;
    source.init([&](uint32_t q) { return q < 8U ? gate + q * stride : up + (q - 8U) * stride; }, r.in.codes_of(row));
    lds_u8* const (&sl)[DEPTH] = slots;
    const float value = sweep_quads<DEPTH>(sl, source, w.hidden / 256U, r.in, row);
    const float other = __shfl_xor(value, 32);
    const bool mine = lane < 32U && p == 0;                   // the lane that publishes feature f0 + rr
    const float g = lane < 32U ? value : other, u = lane < 32U ? other : value;
    float gc = g, uc = u;
    swiglu_clamp(gc, uc, w.swiglu_limit);
    const float h = (gc / (1.0F + exp_of(w.exp_kind, -gc))) * uc;
    const uint32_t at_out = f0 + rr;
    if (mine) {
        if (r.gate_out) r.inter_of(r.gate_out, sidx)[at_out] = g;
        if (r.up_out) r.inter_of(r.up_out, sidx)[at_out] = u;
        if (r.h_out) r.inter_of(r.h_out, sidx)[at_out] = h;
    }
    if (!r.h.codes) return;                               // projection only (the probe form): no A8 image of h
    const int bad = or32_i((mine && !(finite_f(g) && finite_f(u) && finite_f(h))) ? 1 : 0);
    const float amax_wave = max32(mine ? __builtin_fabsf(h) : 0.0F);
    if (lane == 0) { wg_amax[wave] = amax_wave; wg_bad[wave] = bad; }
    __syncthreads();
    if (wg_bad[0] | wg_bad[1] | wg_bad[2] | wg_bad[3]) {
        if (threadIdx.x == 0) {
            atomicOr(r.status_of(row), r.nonfinite_bit);
            atomicOr(r.job_status, static_cast<uint32_t>(MI355_STATUS_NONFINITE_PROJECTION));
        }
        return;
    }
    const float amax = __builtin_fmaxf(__builtin_fmaxf(wg_amax[0], wg_amax[1]), __builtin_fmaxf(wg_amax[2], wg_amax[3]));
    const bool tiny = amax > 0.0F && amax < 0x1p-119F;
    const float dl = (amax == 0.0F || tiny) ? 1.0F : amax / 127.0F;
    const int code = a8_code(h, dl, tiny);
    const int sum_wave = sum32_i(mine ? code : 0);
    if (lane == 0) wg_sum[wave] = sum_wave;
    if (mine) r.h_codes_of(sidx)[at_out] = static_cast<int8_t>(code);
    __syncthreads();
    if (threadIdx.x == 0) {
        r.h_deltas_of(sidx)[grp] = dl;
        r.h_sums_of(sidx)[grp] = wg_sum[0] + wg_sum[1] + wg_sum[2] + wg_sum[3];
    }
}

// The same for Q5_K gate / up tensors (176-byte blocks through the same ring), for every assignment of the item in turn.
template <int DEPTH>
__global__ __launch_bounds__(256) void project_q5k_kernel(mi355_moe_weights w, RowsK r, uint32_t assignments) {
    STRIX_QUAD_SLOTS(DEPTH)
    __shared__ float wg_amax[4];
    __shared__ int wg_sum[4], wg_bad[4];
    const WorkItem item = work_item(w, r, plan_items_at(w.experts, assignments), blockIdx.y);
    const uint32_t e = item.e, begin = item.begin, end = item.end;
    const uint32_t lane = threadIdx.x & 63U, p = lane & 3U, rr = lane >> 2, grp = blockIdx.x;
    const uint32_t f0 = grp * 32U + 8U * wave;
    const size_t base = static_cast<size_t>(e) * w.gate_expert_stride + static_cast<size_t>(f0) * w.gate_row_stride;
    const uint8_t* gate = w.gate + base;
    const uint8_t* up = w.up + base;
    const size_t stride = w.gate_row_stride;
    lds_u8* const (&sl)[DEPTH] = slots;
    const bool mine = lane < 32U && p == 0;                   // the lane that publishes feature f0 + rr
    for (uint32_t a = begin; a < end; ++a) {
        const uint32_t sidx = __builtin_amdgcn_readfirstlane(ordered(r, plan_order_at(w.experts), a)), row = r.row_of(sidx);
        QuadSourceT<11> source;
        source.init([&](uint32_t q) { return q < 8U ? gate + q * stride : up + (q - 8U) * stride; }, r.in.codes_of(row));
        const float value = sweep_quads<DEPTH, true>(sl, source, w.hidden / 256U, r.in, row);
        const float other = __shfl_xor(value, 32);
        const float g = lane < 32U ? value : other, u = lane < 32U ? other : value;
        float gc = g, uc = u;
        swiglu_clamp(gc, uc, w.swiglu_limit);
        const float h = (gc / (1.0F + exp_of(w.exp_kind, -gc))) * uc;
        const uint32_t at_out = f0 + rr;
        if (mine) {
            if (r.gate_out) r.inter_of(r.gate_out, sidx)[at_out] = g;
            if (r.up_out) r.inter_of(r.up_out, sidx)[at_out] = u;
            if (r.h_out) r.inter_of(r.h_out, sidx)[at_out] = h;
        }
        if (!r.h.codes) continue;                         // projection only (the probe form): no A8 image of h
        const int bad = or32_i((mine && !(finite_f(g) && finite_f(u) && finite_f(h))) ? 1 : 0);
        const float amax_wave = max32(mine ? __builtin_fabsf(h) : 0.0F);
        __syncthreads();                                          // the previous assignment's reads of the shared words are done
        if (lane == 0) { wg_amax[wave] = amax_wave; wg_bad[wave] = bad; }
        __syncthreads();
        if (wg_bad[0] | wg_bad[1] | wg_bad[2] | wg_bad[3]) {      // uniform over the workgroup
            if (threadIdx.x == 0) {
                atomicOr(r.status_of(row), r.nonfinite_bit);
                atomicOr(r.job_status, static_cast<uint32_t>(MI355_STATUS_NONFINITE_PROJECTION));
            }
            continue;
        }
        const float amax = __builtin_fmaxf(__builtin_fmaxf(wg_amax[0], wg_amax[1]), __builtin_fmaxf(wg_amax[2], wg_amax[3]));
        const bool tiny = amax > 0.0F && amax < 0x1p-119F;
        const float dl = (amax == 0.0F || tiny) ? 1.0F : amax / 127.0F;
        const int code = a8_code(h, dl, tiny);
        const int sum_wave = sum32_i(mine ? code : 0);
        if (lane == 0) wg_sum[wave] = sum_wave;
        if (mine) r.h_codes_of(sidx)[at_out] = static_cast<int8_t>(code);
        __syncthreads();
        if (threadIdx.x == 0) {
            r.h_deltas_of(sidx)[grp] = dl;
            r.h_sums_of(sidx)[grp] = wg_sum[0] + wg_sum[1] + wg_sum[2] + wg_sum[3];
        }
    }
}

// down rows of one item: a 4-wave workgroup per 64 outputs, 16 per wave.
// Reference: src/cpu/core/routed_expert.cpp:429-447, src/moe_a8_down_contract.cpp:146.
template <int DEPTH>
__global__ __launch_bounds__(256) void down_quad_kernel(mi355_moe_weights w, RowsK r, uint32_t assignments) {
    STRIX_QUAD_SLOTS(DEPTH)
    const WorkItem item = work_item(w, r, plan_items_at(w.experts, assignments), blockIdx.y);
    const uint32_t e = item.e, begin = item.begin, end = item.end;
    if (begin == end) return;
    if (*r.job_status & MI355_STATUS_NONFINITE_PROJECTION) return;
    const uint32_t lane = threadIdx.x & 63U, p = lane & 3U, rr = lane >> 2;
    const uint32_t src = __builtin_amdgcn_readfirstlane(ordered(r, plan_order_at(w.experts), begin));
    const uint32_t o0 = blockIdx.x * 64U + 16U * wave;
    const uint8_t* rows = w.down + static_cast<size_t>(e) * w.down_expert_stride + static_cast<size_t>(o0) * w.down_row_stride;
    const size_t stride = w.down_row_stride;
    QuadSource source;
    source.init([&](uint32_t q) { return rows + q * stride; }, r.h.codes_of(src));
    lds_u8* const (&sl)[DEPTH] = slots;
    const float value = sweep_quads<DEPTH>(sl, source, w.ffn / 256U, r.h, src);
    if (p == 0) r.rawdots_of(src, w.hidden)[o0 + rr] = value;
}

// Ordered combine of the slots of one row. Reference: include/strix/moe/combine.hpp:36-59 (fma form),
// src/ds41_expert_tp.cpp:189-199 (product then add, slots in ascending expert id).
// VEC = columns per thread (4: every row of rawdots / base / output starts on 16 bytes and hidden % 4 == 0). The slots'
// values are all requested before the chain starts, so a thread has top_k loads in flight instead of one.
template <int VEC>
__global__ __launch_bounds__(256) void merge_kernel(mi355_moe_weights w, RowsK r, uint32_t form) {
    typedef float vec_t __attribute__((ext_vector_type(VEC)));
    __shared__ uint32_t slot_order[16];
    __shared__ float slot_weight[16];
    __shared__ uint32_t row_failed;
    const uint32_t row = blockIdx.y, o = (blockIdx.x * 256U + threadIdx.x) * VEC;
    if (threadIdx.x == 0) {
        // fail closed: a row flagged by an earlier stage publishes nothing (the aggregate bit is this kernel's own), and
        // neither does any row of a job whose down phase was skipped (its unweighted outputs are not this job's)
        row_failed = (*r.status_of(row) & ~static_cast<uint32_t>(MI355_STATUS_AGGREGATE)) | (*r.job_status & MI355_STATUS_NONFINITE_PROJECTION);
        for (uint32_t k = 0; k < w.top_k; ++k) slot_order[k] = k;
        if (form == MI355_COMBINE_MULADD_ASCENDING_EXPERT)
            for (uint32_t i = 1; i < w.top_k; ++i)
                for (uint32_t j = i; j > 0 && r.routes_of(row)[slot_order[j]] < r.routes_of(row)[slot_order[j - 1]]; --j) {
                    const uint32_t t = slot_order[j]; slot_order[j] = slot_order[j - 1]; slot_order[j - 1] = t;
                }
        for (uint32_t k = 0; k < w.top_k; ++k) slot_weight[k] = r.route_weights_of(row)[slot_order[k]];
    }
    __syncthreads();
    if (o >= w.hidden || row_failed) return;
    vec_t e[16];
#pragma unroll
    for (uint32_t k = 0; k < 16U; ++k)
        if (k < w.top_k) e[k] = *reinterpret_cast<const vec_t*>(r.rawdots_of(row * w.top_k + slot_order[k], w.hidden) + o);
    vec_t y;
    bool finite = true;
#pragma unroll
    for (int c = 0; c < VEC; ++c) {
        float acc = 0.0F;
#pragma unroll
        for (uint32_t k = 0; k < 16U; ++k) {
            if (k >= w.top_k) continue;
            const float v = e[k][c];
            if (form == MI355_COMBINE_FMA_SLOT_ORDER && k + r.shared_slots < w.top_k) acc = __builtin_fmaf(slot_weight[k], v, acc);
            else acc = acc + slot_weight[k] * v;
        }
        const float out = r.base ? acc + r.base_of(row)[o + c] : acc;
        finite = finite && finite_f(out);
        y[c] = out;
    }
    if (!finite) atomicOr(r.status_of(row), static_cast<uint32_t>(MI355_STATUS_AGGREGATE));
    *reinterpret_cast<vec_t*>(r.output + static_cast<size_t>(row) * r.output_stride + o) = y;
}

constexpr uint32_t kDownMergeSlots = 8;        // top_k bound: 8 waves x 2 ring slots fill the LDS of a compute unit
// Down rows and the ordered combine of a decode batch in one launch: a workgroup owns (row, 64 output columns) and has one
// wave per slot of the row, wave k sweeping the down rows of the expert in slot k (the plan holds one item per assignment,
// in assignment order); the waves leave their 64 values in LDS and wave 0 folds them exactly as merge_kernel does. Only
// waves of one workgroup exchange data, so nothing depends on the visibility of another workgroup's stores.
// Reference: src/cpu/core/routed_expert.cpp:429-447, src/moe_a8_down_contract.cpp:146, include/strix/moe/combine.hpp:36-59.
__global__ __launch_bounds__(64 * kDownMergeSlots) void down_merge_kernel(mi355_moe_weights w, RowsK r, uint32_t assignments, uint32_t form) {
    // the two ring slots are separate LDS objects: the compiler then knows that a copy into one never touches the other and lets
    // the reads of the landed slot go ahead while the next stage's copy is in flight (as slots of one array it waited for both)
    __shared__ __attribute__((aligned(16))) uint8_t ring_even[kDownMergeSlots][slot_bytes(1)];
    __shared__ __attribute__((aligned(16))) uint8_t ring_odd[kDownMergeSlots][slot_bytes(1)];
    __shared__ float slot_value[kDownMergeSlots][64];
    __shared__ uint32_t slot_order[kDownMergeSlots];
    __shared__ float slot_weight[kDownMergeSlots];
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63U, row = blockIdx.y, o = blockIdx.x * 64U + lane;
    uint32_t job;                                                              // (requested together with the item: one round trip, not two)
    uint32_t word[2] = {0U, 0U};
    if (r.awords) {
        if (lane < assignments) word[0] = r.awords[lane];
        if (lane + 64U < assignments) word[1] = r.awords[lane + 64U];
    } else job = *r.job_status;
    const uint32_t a = row * w.top_k + wave;
    const WorkItem item = work_item(w, r, plan_items_at(w.experts, assignments), a);
    const uint32_t e = __builtin_amdgcn_readfirstlane(item.e), begin = __builtin_amdgcn_readfirstlane(item.begin), end = __builtin_amdgcn_readfirstlane(item.end);
    if (r.awords) {
        // a batch planned from early routes: the front launch left its non-finite flags per assignment; every workgroup folds them
        // to the same job word, the first workgroup of a row publishes its row's
        job = (__ballot(word[0] >> 31) | __ballot(word[1] >> 31)) ? static_cast<uint32_t>(MI355_STATUS_NONFINITE_PROJECTION) : 0U;
        if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) r.plan[kPlanLinesAt + kLinesEpoch] += 1U;      // this call's epoch is spent
        if (job && blockIdx.x == 0 && wave == 0) {
            const uint32_t lo = row * w.top_k, hi = lo + w.top_k;
            const bool mine = (lane >= lo && lane < hi && (word[0] >> 31)) || (lane + 64U >= lo && lane + 64U < hi && (word[1] >> 31));
            const bool any = __ballot(mine) != 0;
            if (lane == 0) {
                if (any) atomicOr(r.status_of(row), r.nonfinite_bit);
                atomicOr(r.job_status, static_cast<uint32_t>(MI355_STATUS_NONFINITE_PROJECTION));
            }
        }
    }
    if (job & MI355_STATUS_NONFINITE_PROJECTION) return;                       // the whole job: no down rows, nothing published
    float value = 0.0F;
    if (begin != end) {                                                        // (an invalid route has no item: its row is flagged)
        const uint32_t first = item.first ? item.first - 1U : ordered(r, plan_order_at(w.experts), begin);
        const uint8_t* rows = w.down + static_cast<size_t>(e) * w.down_expert_stride + static_cast<size_t>(blockIdx.x * 64U) * w.down_row_stride;
        const size_t stride = w.down_row_stride;
        lds_u8* const slots[2] = {(lds_u8*)ring_even[wave], (lds_u8*)ring_odd[wave]};
        const uint32_t src[1] = {static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(first))}, lane_rows[1] = {first};
        // (contiguous stages - q4k_blocks.hpp - would be four of 16 rows here instead of three of 64: a wave's time is its number of
        // stage waits, and that form measured 16.9 us against 15.5)
        StageSource source;
        source.init([&](uint32_t q) { return rows + q * stride; });
        const ActRows<1> act(r.h, src, lane_rows);
        float swept[1];
        sweep_rows<1, 2, true>(slots, source, w.ffn / 256U, act, swept);      // narrow codes copies: the slots are slot_bytes(1)
        value = swept[0];
        r.rawdots_of(src[0], w.hidden)[o] = value;
    }
    slot_value[wave][lane] = value;
    if (threadIdx.x == 0) {
        for (uint32_t k = 0; k < w.top_k; ++k) slot_order[k] = k;
        if (form == MI355_COMBINE_MULADD_ASCENDING_EXPERT)
            for (uint32_t i = 1; i < w.top_k; ++i)
                for (uint32_t j = i; j > 0 && r.routes_of(row)[slot_order[j]] < r.routes_of(row)[slot_order[j - 1]]; --j) {
                    const uint32_t t = slot_order[j]; slot_order[j] = slot_order[j - 1]; slot_order[j - 1] = t;
                }
        for (uint32_t k = 0; k < w.top_k; ++k) slot_weight[k] = r.route_weights_of(row)[slot_order[k]];
    }
    __syncthreads();
    // fail closed: a row flagged by an earlier stage publishes nothing (the aggregate bit is the combine's own)
    if (wave != 0 || (*r.status_of(row) & ~static_cast<uint32_t>(MI355_STATUS_AGGREGATE))) return;
    float acc = 0.0F;
    for (uint32_t k = 0; k < w.top_k; ++k) {
        const float ev = slot_value[slot_order[k]][lane];
        if (form == MI355_COMBINE_FMA_SLOT_ORDER && k + r.shared_slots < w.top_k) acc = __builtin_fmaf(slot_weight[k], ev, acc);
        else acc = acc + slot_weight[k] * ev;
    }
    const float y = r.base ? acc + r.base_of(row)[o] : acc;
    if (!finite_f(y)) atomicOr(r.status_of(row), static_cast<uint32_t>(MI355_STATUS_AGGREGATE));
    r.output[static_cast<size_t>(row) * r.output_stride + o] = y;
}

// down_merge_kernel for dense rows of at most four super-blocks (down_row_stride = B * 144): the 64 rows of a column block stream as B
// contiguous stages of 1 KB pieces instead of B stages of 64 separate 144-byte blocks (a read-only launch of this shape moves the
// same bytes in 11.8 us against 14.4 us), the block terms meet in LDS in block order and lane = row adds them in ascending order.
template <int B>
__global__ __launch_bounds__(64 * kDownMergeSlots) void down_merge_flat_kernel(mi355_moe_weights w, RowsK r, uint32_t assignments, uint32_t form) {
    // (the two ring slots are separate LDS objects, as in down_merge_kernel)
    __shared__ __attribute__((aligned(16))) uint8_t ring_even[kDownMergeSlots][kFlatStageBytes];
    __shared__ __attribute__((aligned(16))) uint8_t ring_odd[kDownMergeSlots][kFlatStageBytes];
    __shared__ __attribute__((aligned(16))) uint8_t act_rows[kDownMergeSlots][flat_act_bytes(B)];
    __shared__ float slot_value[kDownMergeSlots][64];
    __shared__ uint32_t slot_order[kDownMergeSlots];
    __shared__ float slot_weight[kDownMergeSlots];
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63U, row = blockIdx.y, o = blockIdx.x * 64U + lane;
    uint32_t job;                                                              // (requested together with the item: one round trip, not two)
    uint32_t word[2] = {0U, 0U};
    if (r.awords) {
        if (lane < assignments) word[0] = r.awords[lane];
        if (lane + 64U < assignments) word[1] = r.awords[lane + 64U];
    } else job = *r.job_status;
    const uint32_t a = row * w.top_k + wave;
    const WorkItem item = work_item(w, r, plan_items_at(w.experts, assignments), a);
    const uint32_t e = __builtin_amdgcn_readfirstlane(item.e), begin = __builtin_amdgcn_readfirstlane(item.begin), end = __builtin_amdgcn_readfirstlane(item.end);
    if (r.awords) {
        // a batch planned from early routes: the front launch left its non-finite flags per assignment; every workgroup folds them
        // to the same job word, the first workgroup of a row publishes its row's
        job = (__ballot(word[0] >> 31) | __ballot(word[1] >> 31)) ? static_cast<uint32_t>(MI355_STATUS_NONFINITE_PROJECTION) : 0U;
        if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) r.plan[kPlanLinesAt + kLinesEpoch] += 1U;      // this call's epoch is spent
        if (job && blockIdx.x == 0 && wave == 0) {
            const uint32_t lo = row * w.top_k, hi = lo + w.top_k;
            const bool mine = (lane >= lo && lane < hi && (word[0] >> 31)) || (lane + 64U >= lo && lane + 64U < hi && (word[1] >> 31));
            const bool any = __ballot(mine) != 0;
            if (lane == 0) {
                if (any) atomicOr(r.status_of(row), r.nonfinite_bit);
                atomicOr(r.job_status, static_cast<uint32_t>(MI355_STATUS_NONFINITE_PROJECTION));
            }
        }
    }
    if (job & MI355_STATUS_NONFINITE_PROJECTION) return;                       // the whole job: no down rows, nothing published
    float value = 0.0F;
    if (begin != end) {                                                        // (an invalid route has no item: its row is flagged)
        const uint32_t first = item.first ? item.first - 1U : ordered(r, plan_order_at(w.experts), begin);
        // the 64 rows of the column block are one run of 64 * B super-blocks: B contiguous stages (q4k_blocks.hpp)
        const uint8_t* rows = w.down + static_cast<size_t>(e) * w.down_expert_stride + static_cast<size_t>(blockIdx.x * 64U) * w.down_row_stride;
        lds_u8* const slots[2] = {(lds_u8*)ring_even[wave], (lds_u8*)ring_odd[wave]};
        const uint32_t src[1] = {static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(first))};
        value = sweep_flat_rows<B, 2>(slots, (lds_u8*)act_rows[wave], rows, r.h, src[0]);
        r.rawdots_of(src[0], w.hidden)[o] = value;
    }
    slot_value[wave][lane] = value;
    if (threadIdx.x == 0) {
        for (uint32_t k = 0; k < w.top_k; ++k) slot_order[k] = k;
        if (form == MI355_COMBINE_MULADD_ASCENDING_EXPERT)
            for (uint32_t i = 1; i < w.top_k; ++i)
                for (uint32_t j = i; j > 0 && r.routes_of(row)[slot_order[j]] < r.routes_of(row)[slot_order[j - 1]]; --j) {
                    const uint32_t t = slot_order[j]; slot_order[j] = slot_order[j - 1]; slot_order[j - 1] = t;
                }
        for (uint32_t k = 0; k < w.top_k; ++k) slot_weight[k] = r.route_weights_of(row)[slot_order[k]];
    }
    __syncthreads();
    // fail closed: a row flagged by an earlier stage publishes nothing (the aggregate bit is the combine's own)
    if (wave != 0 || (*r.status_of(row) & ~static_cast<uint32_t>(MI355_STATUS_AGGREGATE))) return;
    float acc = 0.0F;
    for (uint32_t k = 0; k < w.top_k; ++k) {
        const float ev = slot_value[slot_order[k]][lane];
        if (form == MI355_COMBINE_FMA_SLOT_ORDER && k + r.shared_slots < w.top_k) acc = __builtin_fmaf(slot_weight[k], ev, acc);
        else acc = acc + slot_weight[k] * ev;
    }
    const float y = r.base ? acc + r.base_of(row)[o] : acc;
    if (!finite_f(y)) atomicOr(r.status_of(row), static_cast<uint32_t>(MI355_STATUS_AGGREGATE));
    r.output[static_cast<size_t>(row) * r.output_stride + o] = y;
}


// The same for the smallest decode batches, in the 16-rows-per-wavefront layout of down_quad_kernel: a workgroup owns (row, 16
// output columns), wave k sweeps the 16 down rows of the expert in slot k (lane = (row, pair)), the slots' values meet in LDS
// and the first sixteen lanes of wave 0 fold them as merge_kernel does. One launch instead of two for one to six rows.
template <int DEPTH>
__global__ __launch_bounds__(64 * kDownMergeSlots) void down_merge_quad_kernel(mi355_moe_weights w, RowsK r, uint32_t assignments, uint32_t form) {
    __shared__ __attribute__((aligned(16))) uint8_t mq0[kDownMergeSlots][kQuadSlotBytes];
    __shared__ __attribute__((aligned(16))) uint8_t mq1[kDownMergeSlots][kQuadSlotBytes];
    __shared__ __attribute__((aligned(16))) uint8_t mq2[DEPTH > 2 ? kDownMergeSlots : 1][DEPTH > 2 ? kQuadSlotBytes : 16];
    __shared__ __attribute__((aligned(16))) uint8_t mq3[DEPTH > 3 ? kDownMergeSlots : 1][DEPTH > 3 ? kQuadSlotBytes : 16];
    __shared__ float slot_value[kDownMergeSlots][kQuadRows];
    __shared__ uint32_t slot_order[kDownMergeSlots];
    __shared__ float slot_weight[kDownMergeSlots];
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63U, p = lane & 3U, rr = lane >> 2, row = blockIdx.y, o0 = blockIdx.x * kQuadRows;
    lds_u8* const ring[4] = {(lds_u8*)mq0[wave], (lds_u8*)mq1[wave], (lds_u8*)mq2[DEPTH > 2 ? wave : 0], (lds_u8*)mq3[DEPTH > 3 ? wave : 0]};
    lds_u8* slots[DEPTH];
#pragma unroll
    for (int i = 0; i < DEPTH; ++i) slots[i] = ring[i];
    const uint32_t job = *r.job_status;                                        // (requested together with the item)
    const uint32_t a = row * w.top_k + wave;
    const WorkItem item = work_item(w, r, plan_items_at(w.experts, assignments), a);
    if (job & MI355_STATUS_NONFINITE_PROJECTION) return;                       // the whole job: no down rows, nothing published
    float value = 0.0F;
    if (item.begin != item.end) {                                              // (an invalid route has no item: its row is flagged)
        const uint32_t src = __builtin_amdgcn_readfirstlane(item.first ? item.first - 1U : ordered(r, plan_order_at(w.experts), item.begin));
        const uint8_t* rows = w.down + static_cast<size_t>(item.e) * w.down_expert_stride + static_cast<size_t>(o0) * w.down_row_stride;
        const size_t stride = w.down_row_stride;
        QuadSource source;
        source.init([&](uint32_t q) { return rows + q * stride; }, r.h.codes_of(src));
        lds_u8* const (&sl)[DEPTH] = slots;
        value = sweep_quads<DEPTH>(sl, source, w.ffn / 256U, r.h, src);
        if (p == 0) r.rawdots_of(src, w.hidden)[o0 + rr] = value;
    }
    if (p == 0) slot_value[wave][rr] = value;
    if (threadIdx.x == 0) {
        for (uint32_t k = 0; k < w.top_k; ++k) slot_order[k] = k;
        if (form == MI355_COMBINE_MULADD_ASCENDING_EXPERT)
            for (uint32_t i = 1; i < w.top_k; ++i)
                for (uint32_t j = i; j > 0 && r.routes_of(row)[slot_order[j]] < r.routes_of(row)[slot_order[j - 1]]; --j) {
                    const uint32_t t = slot_order[j]; slot_order[j] = slot_order[j - 1]; slot_order[j - 1] = t;
                }
        for (uint32_t k = 0; k < w.top_k; ++k) slot_weight[k] = r.route_weights_of(row)[slot_order[k]];
    }
    __syncthreads();
    // fail closed: a row flagged by an earlier stage publishes nothing (the aggregate bit is the combine's own)
    if (threadIdx.x >= kQuadRows || (*r.status_of(row) & ~static_cast<uint32_t>(MI355_STATUS_AGGREGATE))) return;
    float acc = 0.0F;
    for (uint32_t k = 0; k < w.top_k; ++k) {
        const float ev = slot_value[slot_order[k]][lane];
        if (form == MI355_COMBINE_FMA_SLOT_ORDER && k + r.shared_slots < w.top_k) acc = __builtin_fmaf(slot_weight[k], ev, acc);
        else acc = acc + slot_weight[k] * ev;
    }
    const uint32_t o = o0 + lane;
    const float y = r.base ? acc + r.base_of(row)[o] : acc;
    if (!finite_f(y)) atomicOr(r.status_of(row), static_cast<uint32_t>(MI355_STATUS_AGGREGATE));
    r.output[static_cast<size_t>(row) * r.output_stride + o] = y;
}

// Down rows + combine in one launch for Q5_1 down rows of whole, 16-byte aligned super-blocks (the host executor's format,
// src/cpu/core/routed_expert.cpp:110-126): the workgroup of (row, 16 columns), wave k = the expert in slot k, each wave with
// the copy ring, the lane layout and the chain order of down_q51_ring_kernel for its one assignment.
template <int DEPTH>
__global__ __launch_bounds__(64 * kDownMergeSlots) void down_merge_q51_kernel(mi355_moe_weights w, RowsK r, uint32_t assignments, uint32_t form) {
    typedef const __attribute__((address_space(3))) u32x4 lds_u32x4;
    typedef const __attribute__((address_space(3))) float lds_f32c;
    typedef const __attribute__((address_space(3))) int32_t lds_i32c;
    constexpr uint32_t kBlock = kQ51Block, RP = group_row_pieces(), WC = group_weight_copies(), PER = WC + 2U;
    // a slot: the 16 rows' 8 groups (3 KB), the one assignment's 256 codes and its [8 deltas][8 sums]
    constexpr uint32_t ROWB = kGroupStage * kBlock, CODES_AT = 1024U * WC, TABLE_AT = CODES_AT + 256U, SLOT = TABLE_AT + 64U;
    static_assert(16U * ROWB == 1024U * WC, "the rows of a stage fill the weight copies");
    __shared__ __attribute__((aligned(16))) uint8_t ring_mem[DEPTH][kDownMergeSlots][SLOT];
    __shared__ float slot_value[kDownMergeSlots][16];
    __shared__ uint32_t slot_order[kDownMergeSlots];
    __shared__ float slot_weight[kDownMergeSlots];
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63U, j = lane & 3U, rr = lane >> 2, row = blockIdx.y;
    const uint32_t o0 = blockIdx.x * 16U, o = o0 + rr;
    const uint32_t job = *r.job_status;                                        // (requested together with the item)
    const WorkItem item = work_item(w, r, plan_items_at(w.experts, assignments), row * w.top_k + wave);
    if (job & MI355_STATUS_NONFINITE_PROJECTION) return;                       // the whole job: no down rows, nothing published
    float value = 0.0F;
    if (item.begin != item.end) {                                              // (an invalid route has no item: its row is flagged)
        const uint32_t src = item.first ? item.first - 1U : ordered(r, plan_order_at(w.experts), item.begin);
        const uint32_t stages = w.ffn / 256U;
        const uint8_t* rows = w.down + static_cast<size_t>(item.e) * w.down_expert_stride + static_cast<size_t>(o0) * w.down_row_stride;
        // the lane's pieces of a stage: piece index i * 64 + lane = row * RP + piece of the row's 8-group segment
        const uint8_t* wsrc[WC];
#pragma unroll
        for (uint32_t i = 0; i < WC; ++i) {
            uint32_t k = i * 64U + lane;
            k = k < 16U * RP ? k : 16U * RP - 1U;                  // padding lanes repeat the last piece into unused LDS
            const uint32_t wr = k / RP, piece = k - RP * wr;
            wsrc[i] = rows + static_cast<size_t>(wr) * w.down_row_stride + 16U * piece;
        }
        // the stage's 256 codes (lanes 0..15) and its [8 deltas][8 sums] (lanes 0..3)
        const uint8_t* csrc = reinterpret_cast<const uint8_t*>(r.h.codes_of(src)) + 16U * (lane & 15U);
        const uint32_t tq = lane & 3U;
        const uint8_t* tsrc = tq < 2U ? reinterpret_cast<const uint8_t*>(r.h.deltas_of(src)) + 16U * tq : reinterpret_cast<const uint8_t*>(r.h.sums_of(src)) + 16U * (tq - 2U);
        const auto start = [&](lds_u8* slot) {
#pragma unroll
            for (uint32_t i = 0; i < WC; ++i) {
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)wsrc[i],
                                                 (__attribute__((address_space(3))) void*)(slot + 1024U * i), 16, 0, 0);
                wsrc[i] += ROWB;
            }
            if (lane < 16U)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)csrc,
                                                 (__attribute__((address_space(3))) void*)(slot + CODES_AT), 16, 0, 0);
            csrc += 256;
            if (lane < 4U)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)tsrc,
                                                 (__attribute__((address_space(3))) void*)(slot + TABLE_AT), 16, 0, 0);
            tsrc += 32;
        };
        lds_u8* ring[DEPTH];
#pragma unroll
        for (int s = 0; s < DEPTH; ++s) ring[s] = (lds_u8*)ring_mem[s][wave];
        float chain = 0.0F;
#pragma unroll
        for (int s = 0; s < DEPTH - 1; ++s)
            if (static_cast<uint32_t>(s) < stages) start(ring[s]);
        for (uint32_t b0 = 0; b0 < stages; b0 += DEPTH) {
#pragma unroll
            for (int s = 0; s < DEPTH; ++s) {
                const uint32_t b = b0 + s;
                if (b < stages) {
                    const uint32_t last = b + DEPTH - 1U < stages ? b + DEPTH - 1U : stages;
                    wait_stages_ahead<PER>(last - 1U - b);
                    if (b + DEPTH - 1U < stages) start(ring[(s + DEPTH - 1) % DEPTH]);
                    const lds_u8* slot = ring[s];
#pragma unroll
                    for (uint32_t c = 0; c < kGroupStage / 4U; ++c) {
                        const uint32_t gl = 4U * c + j;                                 // the lane's group inside the stage
                        float d, m;
                        uint32_t q[8];
                        load_q51_block_lds(slot + rr * ROWB + gl * kBlock, d, m, q);
                        lds_u32x4* codes = (lds_u32x4*)(slot + CODES_AT + 32U * gl);
                        const u32x4 c_lo = codes[0], c_hi = codes[1];
                        const uint32_t cw[8] = {c_lo.x, c_lo.y, c_lo.z, c_lo.w, c_hi.x, c_hi.y, c_hi.z, c_hi.w};
                        int dot = 0;
#pragma unroll
                        for (int i = 0; i < 8; ++i) dot = __builtin_amdgcn_sdot4(static_cast<int>(q[i]), static_cast<int>(cw[i]), dot, false);
                        const float first = d * static_cast<float>(dot);
                        const float combined = first + (m * static_cast<float>(*(lds_i32c*)(slot + TABLE_AT + 32U + 4U * gl)));
                        chain = chain + (*(lds_f32c*)(slot + TABLE_AT + 4U * gl) * combined);
                    }
                }
            }
        }
        value = chain;
        value = value + xor1_f(value);          // chain0 + chain1 | chain2 + chain3
        value = value + xor2_f(value);          // (chain0 + chain1) + (chain2 + chain3)
        if (j == 0) r.rawdots_of(src, w.hidden)[o] = value;
    }
    if (j == 0) slot_value[wave][rr] = value;
    if (threadIdx.x == 0) {
        for (uint32_t k = 0; k < w.top_k; ++k) slot_order[k] = k;
        if (form == MI355_COMBINE_MULADD_ASCENDING_EXPERT)
            for (uint32_t i = 1; i < w.top_k; ++i)
                for (uint32_t jj = i; jj > 0 && r.routes_of(row)[slot_order[jj]] < r.routes_of(row)[slot_order[jj - 1]]; --jj) {
                    const uint32_t t = slot_order[jj]; slot_order[jj] = slot_order[jj - 1]; slot_order[jj - 1] = t;
                }
        for (uint32_t k = 0; k < w.top_k; ++k) slot_weight[k] = r.route_weights_of(row)[slot_order[k]];
    }
    __syncthreads();
    // fail closed: a row flagged by an earlier stage publishes nothing (the aggregate bit is the combine's own)
    if (threadIdx.x >= 16U || (*r.status_of(row) & ~static_cast<uint32_t>(MI355_STATUS_AGGREGATE))) return;
    float sum = 0.0F;
    for (uint32_t k = 0; k < w.top_k; ++k) {
        const float ev = slot_value[slot_order[k]][lane];
        if (form == MI355_COMBINE_FMA_SLOT_ORDER && k + r.shared_slots < w.top_k) sum = __builtin_fmaf(slot_weight[k], ev, sum);
        else sum = sum + slot_weight[k] * ev;
    }
    const uint32_t oc = blockIdx.x * 16U + lane;
    const float y = r.base ? sum + r.base_of(row)[oc] : sum;
    if (!finite_f(y)) atomicOr(r.status_of(row), static_cast<uint32_t>(MI355_STATUS_AGGREGATE));
    r.output[static_cast<size_t>(row) * r.output_stride + oc] = y;
}

// Down rows + combine in one launch for Q6_K down rows (src/moe_a8_down_contract.cpp:147-158): the workgroup of (row, 16 columns),
// wave k = the expert in slot k, lane = (row, pair) with the direct loads and the order of down_q6k_kernel.
__global__ __launch_bounds__(64 * kDownMergeSlots) void down_merge_q6k_kernel(mi355_moe_weights w, RowsK r, uint32_t assignments, uint32_t form) {
    typedef uint32_t u32x4_g __attribute__((ext_vector_type(4)));
    __shared__ float slot_value[kDownMergeSlots][16];
    __shared__ uint32_t slot_order[kDownMergeSlots];
    __shared__ float slot_weight[kDownMergeSlots];
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63U, p = lane & 3U, half = p >> 1, odd = p & 1U, rr = lane >> 2, row = blockIdx.y;
    const uint32_t o = blockIdx.x * 16U + rr;
    const uint32_t job = *r.job_status;                                        // (requested together with the item)
    const WorkItem item = work_item(w, r, plan_items_at(w.experts, assignments), row * w.top_k + wave);
    if (job & MI355_STATUS_NONFINITE_PROJECTION) return;                       // the whole job: no down rows, nothing published
    float value = 0.0F;
    if (item.begin != item.end) {                                              // (an invalid route has no item: its row is flagged)
        const uint32_t src = item.first ? item.first - 1U : ordered(r, plan_order_at(w.experts), item.begin);
        const uint32_t blocks = w.ffn / 256U;
        const uint8_t* wrow = w.down + static_cast<size_t>(item.e) * w.down_expert_stride + static_cast<size_t>(o) * w.down_row_stride;
        const int8_t* h_codes = r.h.codes_of(src);
        const float* h_deltas = r.h.deltas_of(src);
        float acc = 0.0F;
#pragma unroll 2
        for (uint32_t b = 0; b < blocks; ++b) {
            const uint8_t* blk = wrow + static_cast<size_t>(b) * kQ6kBlock;
            uint32_t ql[16], qh[8];
            load_words_2aligned<16>(blk + 64U * half, ql);
            load_words_2aligned<8>(blk + 128U + 32U * half, qh);
            const uint16_t* tail = reinterpret_cast<const uint16_t*>(blk + 192U);
            const uint32_t sc01 = tail[2U * p], sc23 = tail[2U * p + 1U];          // scales 4p, 4p + 1 | 4p + 2, 4p + 3
            const float d = half_bits_to_float(tail[8]);
            const int s[2][2] = {{static_cast<int8_t>(sc01 & 255U), static_cast<int8_t>(sc01 >> 8)},
                                 {static_cast<int8_t>(sc23 & 255U), static_cast<int8_t>(sc23 >> 8)}};
            const u32x4_g* codes = reinterpret_cast<const u32x4_g*>(h_codes + 256U * b + 64U * p);
            const float2 delta = *reinterpret_cast<const float2*>(h_deltas + 8U * b + 2U * p);
            float term[2];
#pragma unroll
            for (uint32_t k = 0; k < 2U; ++k) {
                uint32_t q[8];
#pragma unroll
                for (uint32_t i = 0; i < 8U; ++i) {
                    const uint32_t nibbles = (ql[8U * k + i] >> (4U * odd)) & 0x0f0f0f0fU;
                    const uint32_t pairs = (qh[i] >> (4U * odd + 2U * k)) & 0x03030303U;
                    const uint32_t six = nibbles | (pairs << 4);                   // 0 .. 63 per byte
                    q[i] = ((six | 0x80808080U) - 0x20202020U) ^ 0x80808080U;      // minus 32 per byte, no borrow between bytes
                }
                const u32x4_g c_lo = codes[2U * k], c_hi = codes[2U * k + 1U];
                const uint32_t cw[8] = {c_lo.x, c_lo.y, c_lo.z, c_lo.w, c_hi.x, c_hi.y, c_hi.z, c_hi.w};
                int first = 0, last = 0;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    first = __builtin_amdgcn_sdot4(static_cast<int>(q[i]), static_cast<int>(cw[i]), first, false);
                    last = __builtin_amdgcn_sdot4(static_cast<int>(q[4 + i]), static_cast<int>(cw[4 + i]), last, false);
                }
                const int integer = s[k][0] * first + s[k][1] * last;
                term[k] = (k == 0 ? delta.x : delta.y) * (d * static_cast<float>(integer));
            }
            acc = acc + (term[0] + term[1]);
        }
        value = acc;
        value = value + xor1_f(value);          // acc0 + acc1 | acc2 + acc3
        value = value + xor2_f(value);          // (acc0 + acc1) + (acc2 + acc3)
        if (p == 0) r.rawdots_of(src, w.hidden)[o] = value;
    }
    if (p == 0) slot_value[wave][rr] = value;
    if (threadIdx.x == 0) {
        for (uint32_t k = 0; k < w.top_k; ++k) slot_order[k] = k;
        if (form == MI355_COMBINE_MULADD_ASCENDING_EXPERT)
            for (uint32_t i = 1; i < w.top_k; ++i)
                for (uint32_t jj = i; jj > 0 && r.routes_of(row)[slot_order[jj]] < r.routes_of(row)[slot_order[jj - 1]]; --jj) {
                    const uint32_t t = slot_order[jj]; slot_order[jj] = slot_order[jj - 1]; slot_order[jj - 1] = t;
                }
        for (uint32_t k = 0; k < w.top_k; ++k) slot_weight[k] = r.route_weights_of(row)[slot_order[k]];
    }
    __syncthreads();
    // fail closed: a row flagged by an earlier stage publishes nothing (the aggregate bit is the combine's own)
    if (threadIdx.x >= 16U || (*r.status_of(row) & ~static_cast<uint32_t>(MI355_STATUS_AGGREGATE))) return;
    float sum = 0.0F;
    for (uint32_t k = 0; k < w.top_k; ++k) {
        const float ev = slot_value[slot_order[k]][lane];
        if (form == MI355_COMBINE_FMA_SLOT_ORDER && k + r.shared_slots < w.top_k) sum = __builtin_fmaf(slot_weight[k], ev, sum);
        else sum = sum + slot_weight[k] * ev;
    }
    const uint32_t oc = blockIdx.x * 16U + lane;
    const float y = r.base ? sum + r.base_of(row)[oc] : sum;
    if (!finite_f(y)) atomicOr(r.status_of(row), static_cast<uint32_t>(MI355_STATUS_AGGREGATE));
    r.output[static_cast<size_t>(row) * r.output_stride + oc] = y;
}

// Down rows + combine in one launch for Q8_0 down tensors (the host executor's format, src/cpu/core/routed_expert.cpp:110-126): the
// workgroup of (row, 16 columns) again, wave k = the expert in slot k, lane = (row, chain) with the direct block loads and the
// chain order of down_groups_kernel<0>; one item per assignment (the fused decode router's plan).
__global__ __launch_bounds__(64 * kDownMergeSlots) void down_merge_q8_0_kernel(mi355_moe_weights w, RowsK r, uint32_t assignments, uint32_t form) {
    typedef uint32_t u32x4_g __attribute__((ext_vector_type(4)));
    __shared__ float slot_value[kDownMergeSlots][16];
    __shared__ uint32_t slot_order[kDownMergeSlots];
    __shared__ float slot_weight[kDownMergeSlots];
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63U, j = lane & 3U, odd = j & 1U, rr = lane >> 2, row = blockIdx.y;
    const uint32_t o = blockIdx.x * 16U + rr;
    const uint32_t job = *r.job_status;                                        // (requested together with the item)
    const WorkItem item = work_item(w, r, plan_items_at(w.experts, assignments), row * w.top_k + wave);
    if (job & MI355_STATUS_NONFINITE_PROJECTION) return;                       // the whole job: no down rows, nothing published
    float value = 0.0F;
    if (item.begin != item.end) {                                              // (an invalid route has no item: its row is flagged)
        const uint32_t src = item.first ? item.first - 1U : ordered(r, plan_order_at(w.experts), item.begin);
        const uint32_t per_chain = w.ffn / 128U;
        const uint8_t* wrow = w.down + static_cast<size_t>(item.e) * w.down_expert_stride + static_cast<size_t>(o) * w.down_row_stride + 34U * j;
        const int8_t* h_codes = r.h.codes_of(src);
        const float* h_deltas = r.h.deltas_of(src);
        float chain = 0.0F;
#pragma unroll 2
        for (uint32_t c = 0; c < per_chain; ++c) {
            const uint32_t g = 4U * c + j;
            float d, m;
            uint32_t q[8];
            load_group_block<0>(wrow + static_cast<size_t>(c) * (4U * 34U), odd, d, m, q);
            const u32x4_g* codes = reinterpret_cast<const u32x4_g*>(h_codes + 32U * g);
            const u32x4_g c_lo = codes[0], c_hi = codes[1];
            const uint32_t cw[8] = {c_lo.x, c_lo.y, c_lo.z, c_lo.w, c_hi.x, c_hi.y, c_hi.z, c_hi.w};
            int dot = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) dot = __builtin_amdgcn_sdot4(static_cast<int>(q[i]), static_cast<int>(cw[i]), dot, false);
            chain = chain + (h_deltas[g] * (d * static_cast<float>(dot)));
        }
        value = chain;
        value = value + xor1_f(value);          // chain0 + chain1 | chain2 + chain3
        value = value + xor2_f(value);          // (chain0 + chain1) + (chain2 + chain3)
        if (j == 0) r.rawdots_of(src, w.hidden)[o] = value;
    }
    if (j == 0) slot_value[wave][rr] = value;
    if (threadIdx.x == 0) {
        for (uint32_t k = 0; k < w.top_k; ++k) slot_order[k] = k;
        if (form == MI355_COMBINE_MULADD_ASCENDING_EXPERT)
            for (uint32_t i = 1; i < w.top_k; ++i)
                for (uint32_t jj = i; jj > 0 && r.routes_of(row)[slot_order[jj]] < r.routes_of(row)[slot_order[jj - 1]]; --jj) {
                    const uint32_t t = slot_order[jj]; slot_order[jj] = slot_order[jj - 1]; slot_order[jj - 1] = t;
                }
        for (uint32_t k = 0; k < w.top_k; ++k) slot_weight[k] = r.route_weights_of(row)[slot_order[k]];
    }
    __syncthreads();
    // fail closed: a row flagged by an earlier stage publishes nothing (the aggregate bit is the combine's own)
    if (threadIdx.x >= 16U || (*r.status_of(row) & ~static_cast<uint32_t>(MI355_STATUS_AGGREGATE))) return;
    float acc = 0.0F;
    for (uint32_t k = 0; k < w.top_k; ++k) {
        const float ev = slot_value[slot_order[k]][lane];
        if (form == MI355_COMBINE_FMA_SLOT_ORDER && k + r.shared_slots < w.top_k) acc = __builtin_fmaf(slot_weight[k], ev, acc);
        else acc = acc + slot_weight[k] * ev;
    }
    const uint32_t oc = blockIdx.x * 16U + lane;
    const float y = r.base ? acc + r.base_of(row)[oc] : acc;
    if (!finite_f(y)) atomicOr(r.status_of(row), static_cast<uint32_t>(MI355_STATUS_AGGREGATE));
    r.output[static_cast<size_t>(row) * r.output_stride + oc] = y;
}

// SwiGLU + A8 re-quantisation of dense gate/up rows. Reference: src/cpu/core/routed_expert.cpp:147-170.
__global__ __launch_bounds__(256) void swiglu_quantize_kernel(const float* gate, const float* up, uint32_t ffn, uint32_t exp_kind, float limit,
                                                              int8_t* codes, float* deltas, int32_t* sums, float* h_out, uint32_t* status,
                                                              uint32_t* job_status) {
    const uint32_t row = blockIdx.y, groups = ffn / 32U, grp = blockIdx.x * 8U + (threadIdx.x >> 5), l = threadIdx.x & 31U;
    if (grp >= groups) return;
    const size_t at = static_cast<size_t>(row) * ffn + grp * 32U + l;
    const float g = gate[at], u = up[at];
    float gc = g, uc = u;
    swiglu_clamp(gc, uc, limit);
    const float ex = exp_of(exp_kind, -gc);
    const float hv = (gc / (1.0F + ex)) * uc;
    if (h_out) h_out[at] = hv;
    const int bad = or32_i((finite_f(g) && finite_f(u) && finite_f(hv)) ? 0 : 1);
    if (bad) {
        if (l == 0 && status) atomicOr(&status[row], static_cast<uint32_t>(MI355_STATUS_NONFINITE_PROJECTION));
        if (l == 0 && job_status) atomicOr(job_status, static_cast<uint32_t>(MI355_STATUS_NONFINITE_PROJECTION));
        return;
    }
    const float amax = max32(__builtin_fabsf(hv));
    const bool tiny = amax > 0.0F && amax < 0x1p-119F;
    const float dl = (amax == 0.0F || tiny) ? 1.0F : amax / 127.0F;
    const int code = a8_code(hv, dl, tiny);
    const int sum = sum32_i(code);
    codes[at] = static_cast<int8_t>(code);
    if (l == 0) {
        deltas[static_cast<size_t>(row) * groups + grp] = dl;
        sums[static_cast<size_t>(row) * groups + grp] = sum;
    }
}

// A property of the current device, asked once per device ordinal (0 if the runtime cannot say).
inline uint32_t device_property(hipDeviceAttribute_t what, std::atomic<uint32_t> (&known)[64]) {
    int device = 0, value = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0) return 0;
    if (device < 64) {
        const uint32_t seen = known[device].load(std::memory_order_relaxed);
        if (seen != 0) return seen;
    }
    if (hipDeviceGetAttribute(&value, what, device) != hipSuccess || value <= 0) return 0;
    if (device < 64) known[device].store(static_cast<uint32_t>(value), std::memory_order_relaxed);
    return static_cast<uint32_t>(value);
}
inline uint32_t compute_units() {
    static std::atomic<uint32_t> known[64];
    return device_property(hipDeviceAttributeMultiprocessorCount, known);
}
// LDS bytes of one compute unit
inline uint32_t lds_per_unit() {
    static std::atomic<uint32_t> known[64];
    return device_property(hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, known);
}
// wavefronts of a launch that are all resident at once when each holds `lds_each` bytes of LDS
inline uint64_t resident_waves(uint32_t lds_each) {
    return static_cast<uint64_t>(compute_units()) * (lds_per_unit() / lds_each);
}

// ======================================================================================================== dispatch
// Up to 4 (routed experts) or 8 (dense matrix) activation rows share one sweep of an expert's weights; an expert with
// more assignments is swept again for the rest.
// Ring depth: the deepest of 4, 3, 2 at which every workgroup of the launch is resident at once (LDS is what limits it).
inline int ring_depth(uint64_t waves, int nbmax) {
    for (int d = 4; d > 2; --d)
        if (waves <= resident_waves(static_cast<uint32_t>(d) * slot_bytes(nbmax))) return d;
    return 2;
}
template <int NBMAX>
inline void launch_project_nb(const mi355_moe_weights& w, const RowsK& r, uint32_t rows, dim3 grid, hipStream_t st) {
    switch (ring_depth(static_cast<uint64_t>(grid.x) * grid.y, NBMAX)) {
    case 4: project_wave_kernel<NBMAX, 4><<<grid, 64, 0, st>>>(w, r, rows * w.top_k); break;
    case 3: project_wave_kernel<NBMAX, 3><<<grid, 64, 0, st>>>(w, r, rows * w.top_k); break;
    default: project_wave_kernel<NBMAX, 2><<<grid, 64, 0, st>>>(w, r, rows * w.top_k); break;
    }
}
template <int NBMAX>
inline void launch_down_nb(const mi355_moe_weights& w, const RowsK& r, uint32_t rows, dim3 grid, hipStream_t st) {
    switch (ring_depth(static_cast<uint64_t>(grid.x) * grid.y, NBMAX)) {
    case 4: down_wave_kernel<NBMAX, 4><<<grid, 64, 0, st>>>(w, r, rows * w.top_k); break;
    case 3: down_wave_kernel<NBMAX, 3><<<grid, 64, 0, st>>>(w, r, rows * w.top_k); break;
    default: down_wave_kernel<NBMAX, 2><<<grid, 64, 0, st>>>(w, r, rows * w.top_k); break;
    }
}
inline RowsK rows_k(const mi355_moe_rows& r, const mi355_moe_weights& w) {
    RowsK k{};
    static_cast<mi355_moe_rows&>(k) = r;
    k.slot_stride = w.ffn;
    k.top_k = w.top_k;
    k.nonfinite_bit = MI355_STATUS_NONFINITE_PROJECTION;
    k.in = dense_image(r.codes, r.deltas, r.sums, w.hidden);
    k.h = dense_image(r.down_codes, r.down_deltas, r.down_sums, w.ffn);
    k.routes_rs = k.route_weights_rs = 4ULL * w.top_k;
    k.status_rs = 4;
    k.inter_rs = 4ULL * w.top_k * w.ffn;
    k.rawdots_rs = 4ULL * w.top_k * w.hidden;
    k.base_rs = 4ULL * w.hidden;
    return k;
}
// every per-row view back to back (the layouts of mi355_moe_rows): the forms that read the fields as plain arrays apply
inline bool dense_rows(const RowsK& k, const mi355_moe_weights& w) {
    return !k.assignments && !k.in.table && k.in.per_row == 1U && k.in.codes_rs == w.hidden && k.in.deltas_rs == w.hidden / 8U && k.in.sums_rs == w.hidden / 8U &&
           k.h.per_row == 1U && k.h.codes_rs == w.ffn && k.h.deltas_rs == w.ffn / 8U && k.h.sums_rs == w.ffn / 8U && k.slot_stride == w.ffn &&
           k.inter_rs == 4ULL * w.top_k * w.ffn && k.rawdots_rs == 4ULL * w.top_k * w.hidden && k.status_rs == 4;
}

// ---- dense matrix (one expert, every row uses it): the pair-per-lane sweep ------------------------------------------
template <int NA, int AL, int KL = 1>
inline void launch_pairs_depth(const PairArgs& a, uint32_t matrices, hipStream_t st) {
    const dim3 grid(a.rows / pair_rows<AL, KL>(), matrices);
    const uint64_t waves = static_cast<uint64_t>(grid.x) * grid.y;
    // 4 slots when every wavefront of the launch is resident with them and the wait counter can express 3 stages ahead
    const bool deep = 3U * pair_copies<NA, AL, KL>() <= 63U && waves <= resident_waves(4U * pair_slot_bytes<NA, AL, KL>());
    if (deep) q4k_pairs_kernel<NA, AL, 4, KL><<<grid, 64, 0, st>>>(a);
    else q4k_pairs_kernel<NA, AL, 2, KL><<<grid, 64, 0, st>>>(a);
}
// nacts <= 8 activation rows. A matrix with few rows gives few wavefronts, each with a long instruction stream (the whole
// of K): such launches spread every row over more lanes - the four super-blocks of a stage over a quad and, with >= 4
// activation rows, two activation lanes - which multiplies the wavefronts and divides each one's instruction stream.
inline void launch_pairs(const PairArgs& a, uint32_t matrices, hipStream_t st) {
    const bool narrow = static_cast<uint64_t>(a.rows) * matrices < 16384U;
    if (a.nacts <= 1U) { if (narrow) launch_pairs_depth<1, 1, 4>(a, matrices, st); else launch_pairs_depth<1, 1>(a, matrices, st); }
    else if (a.nacts <= 2U) { if (narrow) launch_pairs_depth<2, 1, 4>(a, matrices, st); else launch_pairs_depth<2, 1>(a, matrices, st); }
    else if (a.nacts <= 4U) { if (narrow) launch_pairs_depth<2, 2, 4>(a, matrices, st); else launch_pairs_depth<4, 1>(a, matrices, st); }
    else { if (narrow) launch_pairs_depth<4, 2, 4>(a, matrices, st); else launch_pairs_depth<8, 1>(a, matrices, st); }
}
// The dense form needs fp32 gate / up rows as workspace (the optional intermediates views) because a wavefront holds
// 16 rows, not a whole 32-output SwiGLU group.
inline bool dense_pairs_ok(const mi355_moe_weights& w, uint32_t rows) {
    return w.gate_type == MI355_TYPE_Q4_K && w.down_type == MI355_TYPE_Q4_K &&
           w.experts == 1U && w.top_k == 1U && rows <= 8U && (w.hidden / 256U) % kPairBlocks == 0 && (w.ffn / 256U) % kPairBlocks == 0 &&
           w.gate_row_stride < (1ULL << 24) && w.down_row_stride < (1ULL << 24);
}
inline void launch_project_dense(const mi355_moe_weights& w, const RowsK& r, uint32_t rows, hipStream_t st) {
    PairArgs a{};
    a.m[0] = PairMatrix{w.gate, w.gate_row_stride, r.gate_out, w.ffn};
    a.m[1] = PairMatrix{w.up, w.gate_row_stride, r.up_out, w.ffn};
    a.rows = w.ffn; a.blocks = w.hidden / 256U; a.img = r.in; a.nacts = rows;
    launch_pairs(a, 2, st);
    swiglu_quantize_kernel<<<dim3((w.ffn / 32U + 7U) / 8U, rows), 256, 0, st>>>(r.gate_out, r.up_out, w.ffn, w.exp_kind, w.swiglu_limit, r.down_codes, r.down_deltas,
                                                                                r.down_sums, r.h_out, r.status, r.job_status);
}
inline void launch_down_dense(const mi355_moe_weights& w, const RowsK& r, uint32_t rows, hipStream_t st) {
    PairArgs a{};
    a.m[0] = PairMatrix{w.down, w.down_row_stride, r.rawdots, w.hidden};
    a.rows = w.hidden; a.blocks = w.ffn / 256U; a.img = r.h; a.nacts = rows;
    a.skip_flag = r.job_status; a.skip_mask = MI355_STATUS_NONFINITE_PROJECTION;
    a.publish = r;                 // (r.top1_form != 0: the launch publishes the rows' outputs as well)
    launch_pairs(a, 1, st);
}

// ---- work items of 3..32 rows on the int8 matrix cores (q4k_mma_moe.hpp) ---------------------------------------------
// A dense Q4_K FFN (one expert, top-1, assignment i = row i) with at least 3 rows, in chunks of the sweep's width.
inline bool mma_dense(const mi355_moe_weights& w, const RowsK& r, uint32_t rows) {
    return w.gate_type == MI355_TYPE_Q4_K && w.down_type == MI355_TYPE_Q4_K && w.experts == 1U && w.top_k == 1U && rows >= 3U && !r.assignments;
}
// Routed experts of a batch past the decode sizes whose experts hold several rows each on average: the plan cuts an expert's
// rows into items of this many (0: the vector-ALU sweeps serve the batch).
// Items of up to four 32-row sweeps: the later sweeps of a tile's weights hit the cache, and an expert with thousands of rows
// still spreads over many workgroups.
constexpr uint32_t kMmaItemRows = 128;
inline uint32_t mma_grouped_split(const mi355_moe_weights& w, uint32_t rows) {
    if (w.gate_type != MI355_TYPE_Q4_K || w.down_type != MI355_TYPE_Q4_K || w.experts == 1U || rows <= kFusedMaxRows) return 0U;
    const uint64_t assignments = static_cast<uint64_t>(rows) * w.top_k;
    return assignments >= 16ULL * w.experts ? kMmaItemRows : assignments >= 4ULL * w.experts ? 16U : 0U;
}
template <int NAL>
inline void launch_mma_project_nal(const mi355_moe_weights& w, const RowsK& r, uint32_t rows, uint32_t dense, uint32_t items, hipStream_t st) {
    const dim3 grid(w.ffn / 32U, dense ? (dense + 2U * NAL - 1U) / (2U * NAL) : items);
    q4k_mma_project_kernel<NAL, (NAL >= 8 ? 2 : 3)><<<grid, 256, 0, st>>>(w, r, rows * w.top_k, dense);
}
// A launch with no more workgroups than compute units (few, long rows) runs four stages of a tile at a time (measured at 5120
// rows x 27648, 8 rows: 59 -> 33 us; ring depths 2..4 within 2 us of each other in both forms).
template <int NAL>
inline void launch_mma_down_nal(const mi355_moe_weights& w, const RowsK& r, uint32_t rows, uint32_t dense, uint32_t items, hipStream_t st) {
    const dim3 grid(w.hidden / kMmaRows, dense ? (dense + 2U * NAL - 1U) / (2U * NAL) : items);
    if constexpr (NAL <= 8) {
        if (static_cast<uint64_t>(grid.x) * grid.y <= compute_units()) {
            q4k_mma_down_kernel<NAL, 2, 4><<<grid, 1024, 0, st>>>(w, r, rows * w.top_k, dense);
            return;
        }
    }
    q4k_mma_down_kernel<NAL, (NAL >= 8 ? 2 : 3), 1><<<grid, 256, 0, st>>>(w, r, rows * w.top_k, dense);
}
// width: the most rows an item (or the dense batch) holds
inline void launch_mma_project(const mi355_moe_weights& w, const RowsK& r, uint32_t rows, uint32_t dense, uint32_t items, uint32_t width, hipStream_t st) {
    if (width <= 4U) launch_mma_project_nal<2>(w, r, rows, dense, items, st);
    else if (width <= 8U) launch_mma_project_nal<4>(w, r, rows, dense, items, st);
    else if (width <= 16U) launch_mma_project_nal<8>(w, r, rows, dense, items, st);
    else launch_mma_project_nal<16>(w, r, rows, dense, items, st);
}
// A dense FFN's gate and up rows as raw values into the intermediates, then the SwiGLU / A8 kernel (5..16 rows, one chunk).
inline void launch_mma_gate_up(const mi355_moe_weights& w, const RowsK& r, uint32_t rows, hipStream_t st) {
    const dim3 grid(w.ffn / kMmaRows, 1, 2);
    if (rows <= 8U) q4k_mma_down_kernel<4, 3, 1, true><<<grid, 256, 0, st>>>(w, r, rows, rows);
    else q4k_mma_down_kernel<8, 2, 1, true><<<grid, 256, 0, st>>>(w, r, rows, rows);
    swiglu_quantize_kernel<<<dim3((w.ffn / 32U + 7U) / 8U, rows), 256, 0, st>>>(r.gate_out, r.up_out, w.ffn, w.exp_kind, w.swiglu_limit, r.down_codes, r.down_deltas,
                                                                                r.down_sums, r.h_out, r.status, r.job_status);
}
// (the down rows run best 16 rows to a sweep: 4096 rows over 256 experts, hidden 4096 / ffn 2048: 2.57 ms against 3.03 ms with 32)
inline void launch_mma_down(const mi355_moe_weights& w, const RowsK& r, uint32_t rows, uint32_t dense, uint32_t items, uint32_t width, hipStream_t st) {
    if (width <= 4U) launch_mma_down_nal<2>(w, r, rows, dense, items, st);
    else if (width <= 8U) launch_mma_down_nal<4>(w, r, rows, dense, items, st);
    else launch_mma_down_nal<8>(w, r, rows, dense, items, st);
}

inline void launch_plan(RoutesView routes, uint32_t experts, uint32_t assignments, uint32_t split, uint32_t bound, uint32_t* plan,
                        hipStream_t st) {
    // plan_kernel's own order fill is one thread per expert walking every assignment: fine for a decode batch, far too slow
    // beyond a few hundred assignments (4096 assignments of one expert: 0.55 ms), where a wave per expert does it instead
    const bool large = assignments > 256U;
    plan_kernel<<<1, 1024, 0, st>>>(routes, experts, assignments, split, bound, large ? 0U : 1U, plan);
    if (large) plan_order_kernel<<<experts, 1024, 0, st>>>(routes, experts, assignments, plan);
}
// Decode batches of at most this many assignments (six tokens at top-8) run the 16-rows-per-wavefront sweep (q4k_quads.hpp),
// with a 4-slot ring up to 16 assignments and a 2-slot ring above (every workgroup of the launch stays resident); measured
// at hidden 2048 / ffn 768: faster than the 64-row sweep up to 48 assignments, slower at 64. Such a batch is planned one
// assignment per item (the fused router's plan, and the staged plan with pieces of one).
constexpr uint32_t kQuadMaxItems = 48;
inline bool quad_sweep(const mi355_moe_weights& w, uint32_t rows) {
    return rows <= kFusedMaxRows && rows * w.top_k <= kQuadMaxItems && w.experts > 1U;
}
// grouped: the plan's items hold several assignments (the one-assignment sweeps do not apply)
inline void launch_project(const mi355_moe_weights& w, const RowsK& r, uint32_t rows, uint32_t umax, hipStream_t st, bool grouped = false) {
    if (w.gate_type == MI355_TYPE_Q5_K) {
        // the deepest ring at which every workgroup of the launch is resident (4 waves x DEPTH x 4 KB each)
        const uint64_t groups = static_cast<uint64_t>(w.ffn / 32U) * umax;
        if (groups * 4U <= resident_waves(4U * kQuadSlotBytes)) project_q5k_kernel<4><<<dim3(w.ffn / 32U, umax), 256, 0, st>>>(w, r, rows * w.top_k);
        else project_q5k_kernel<2><<<dim3(w.ffn / 32U, umax), 256, 0, st>>>(w, r, rows * w.top_k);
        return;
    }
    if (!grouped && quad_sweep(w, rows)) {
        const uint32_t items = rows * w.top_k;
        if (items <= 16U) project_quad_kernel<4><<<dim3(w.ffn / 32U, items), 256, 0, st>>>(w, r, items);
        else project_quad_kernel<2><<<dim3(w.ffn / 32U, items), 256, 0, st>>>(w, r, items);
        return;
    }
    if (mma_dense(w, r, rows)) {
        if (rows > 4U && rows <= 16U && r.gate_out && r.up_out && dense_rows(r, w)) return launch_mma_gate_up(w, r, rows, st);
        return launch_mma_project(w, r, rows, rows, 0, rows, st);
    }
    if (const uint32_t split = mma_grouped_split(w, rows); split && r.plan) return launch_mma_project(w, r, rows, 0, umax, split, st);
    if (dense_pairs_ok(w, rows) && dense_rows(r, w) && r.gate_out && r.up_out) return launch_project_dense(w, r, rows, st);
    const dim3 grid(w.ffn / 32U, umax);
    if (w.experts == 1U && rows > 4U) launch_project_nb<8>(w, r, rows, grid, st);
    else launch_project_nb<4>(w, r, rows, grid, st);
}
// Returns true when the launch also published the output rows (a dense top-1 job with r.top1_form set: the two dense sweeps).
inline bool launch_down(const mi355_moe_weights& w, const RowsK& r, uint32_t rows, uint32_t umax, hipStream_t st, bool grouped = false) {
    if (w.down_type != MI355_TYPE_Q4_K) {      // Q8_0 / Q5_1 (blocks of 32, four chains per row) and Q6_K (pairs per super-block)
        const uint32_t assignments = rows * w.top_k, items_at = plan_items_at(w.experts, assignments), order_at = plan_order_at(w.experts);
        const dim3 grid(w.hidden / kDownGroupsRows, umax);
        // Q5_1 rows of whole super-blocks at 16-byte aligned addresses stream through a copy ring (its depth by residency)
        if (w.down_type == MI355_TYPE_Q5_1 && w.ffn % 256U == 0 && w.down_row_stride % 16U == 0 && w.down_expert_stride % 16U == 0) {
            if (static_cast<uint64_t>(grid.x) * grid.y * 4U <= resident_waves(4U * group_slot_bytes())) down_q51_ring_kernel<4><<<grid, 256, 0, st>>>(w, r, assignments, items_at, order_at);
            else down_q51_ring_kernel<2><<<grid, 256, 0, st>>>(w, r, assignments, items_at, order_at);
        }
        else if (w.down_type == MI355_TYPE_Q8_0) down_groups_kernel<0><<<grid, 256, 0, st>>>(w, r, assignments, items_at, order_at);
        else if (w.down_type == MI355_TYPE_Q5_1) down_groups_kernel<1><<<grid, 256, 0, st>>>(w, r, assignments, items_at, order_at);
        else launch_down_q6k(w, r, grid, assignments, items_at, order_at, st);
        return false;
    }
    if (!grouped && quad_sweep(w, rows)) {
        const uint32_t items = rows * w.top_k;
        if (items <= 16U) down_quad_kernel<4><<<dim3(w.hidden / 64U, items), 256, 0, st>>>(w, r, items);
        else down_quad_kernel<2><<<dim3(w.hidden / 64U, items), 256, 0, st>>>(w, r, items);
        return false;
    }
    if (mma_dense(w, r, rows)) { launch_mma_down(w, r, rows, rows, 0, rows, st); return r.top1_form != 0; }
    RowsK plain = r;
    plain.top1_form = 0;
    if (const uint32_t split = mma_grouped_split(w, rows); split && r.plan) { launch_mma_down(w, plain, rows, 0, umax, split, st); return false; }
    if (dense_pairs_ok(w, rows) && dense_rows(r, w)) { launch_down_dense(w, r, rows, st); return r.top1_form != 0; }
    const dim3 grid(w.hidden / 64U, umax);
    if (w.experts == 1U && rows > 4U) launch_down_nb<8>(w, r, rows, grid, st);
    else launch_down_nb<4>(w, r, rows, grid, st);
    return false;
}
// An expert's assignments are cut into work items of at most `split` rows: a wave's instruction stream grows with every
// activation row it serves while its weight stream does not, so wide items finish last; the second read of a split
// expert's weights comes from the last-level cache. A dense matrix: every row shares one sweep.
inline uint32_t plan_split(const mi355_moe_weights& w, uint32_t rows) {
    if (w.experts == 1U) return 8;
    if (const uint32_t split = mma_grouped_split(w, rows)) return split;     // items for the matrix-core sweep
    if (rows > kFusedMaxRows) return 4U;
    if (quad_sweep(w, rows)) return 1U;       // the 16-rows-per-wavefront sweep serves one assignment per item
    // decode batches: one item per assignment while an expert's gate + up rows are a few MB (the second sweep of an expert
    // that two rows chose is a cache hit and the short instruction streams finish sooner); larger experts are swept once
    // for every two rows that chose them (hidden 6144, ffn 1280, 16 rows: 384 -> 351 us)
    const uint64_t sweep_bytes = 2ULL * w.ffn * (w.hidden / 256U) * kQ4kBlock;
    return sweep_bytes >= (4ULL << 20) ? 2U : 1U;
}
inline uint32_t item_bound(const mi355_moe_weights& w, uint32_t rows) {
    return plan_item_bound(w.experts, rows * w.top_k, plan_split(w, rows));
}

// ======================================================================================================== admission
// bytes of a GGUF row of k weights (k a multiple of 256)
inline uint64_t moe_row_bytes(uint32_t type, uint32_t k) {
    if (type == MI355_TYPE_Q8_0) return static_cast<uint64_t>(k / 32U) * kQ80Block;
    if (type == MI355_TYPE_Q5_1) return static_cast<uint64_t>(k / 32U) * 24U;
    if (type == MI355_TYPE_Q5_K) return static_cast<uint64_t>(k / 256U) * kQ5kBlock;
    if (type == MI355_TYPE_Q6_K) return static_cast<uint64_t>(k / 256U) * kQ6kBlock;
    return static_cast<uint64_t>(k / 256U) * kQ4kBlock;
}

// Tensor formats by arithmetic class. Integer-dot entries: gate/up Q4_K or Q5_K; down Q4_K, the host executor's Q8_0 /
// Q5_1 (src/cpu/core/routed_expert.hpp:27-28) or Q6_K (src/moe_a8_down_contract.cpp:147). The matrix-core prefill form: Q4_K, Q5_K or Q8_0 for either (a dense shared
// expert is experts = top_k = 1). The merge reads no weights.
enum MoeClass { kIntegerClass, kPrefillClass, kAnyClass };
int32_t check_moe(const mi355_moe_weights* w, const mi355_moe_rows* r, uint32_t rows, mi355_moe_weights& wv, MoeClass cls = kIntegerClass,
                  bool need_tensors = true) {
    STRIX_REQUIRE(w && r, "moe: null weights or rows");
    STRIX_REQUIRE(rows > 0, "moe: rows must be positive");
    const bool gate_q8 = w->gate_type == MI355_TYPE_Q8_0, down_q8 = w->down_type == MI355_TYPE_Q8_0;
    const bool down_q51 = w->down_type == MI355_TYPE_Q5_1 || w->down_type == MI355_TYPE_Q6_K;      // integer class only
    STRIX_REQUIRE(w->gate_type == MI355_TYPE_Q4_K || w->gate_type == MI355_TYPE_Q5_K || (gate_q8 && cls != kIntegerClass),
                  cls == kPrefillClass ? "moe prefill: gate/up weights must be Q4_K (type 12), Q5_K (type 13) or Q8_0 (type 8)" : "moe: gate/up weights must be Q4_K (type 12) or Q5_K (type 13)");
    if (!(w->down_type == MI355_TYPE_Q4_K || down_q8 || (down_q51 && cls != kPrefillClass) || (w->down_type == MI355_TYPE_Q5_K && cls != kIntegerClass)))
        return fail(MI355_E_UNSUPPORTED, cls == kPrefillClass ? "moe prefill: down weights must be Q4_K (type 12), Q5_K (type 13) or Q8_0 (type 8)"
                                                               : "moe: down weights must be Q4_K (type 12), Q8_0 (type 8), Q5_1 (type 7) or Q6_K (type 14)");
    STRIX_REQUIRE(w->hidden >= 256 && w->hidden % 256U == 0, "moe: hidden must be a positive multiple of 256");
    // K-quant down rows are super-blocks of 256; the executor's block-of-32 formats need four chains of groups (src/cpu/core/routed_expert.hpp:22)
    const uint32_t ffn_unit = (cls != kPrefillClass && (down_q8 || w->down_type == MI355_TYPE_Q5_1)) ? 128U : 256U;
    STRIX_REQUIRE(w->ffn >= ffn_unit && w->ffn % ffn_unit == 0, "moe: ffn must be a positive multiple of 256 (Q8_0 / Q5_1 down rows: 128)");
    STRIX_REQUIRE(w->experts > 0 && w->experts <= kRouteMaxExperts, "moe: experts must be within 1..1024");
    STRIX_REQUIRE(w->top_k > 0 && w->top_k <= kRouteMaxTopK && w->top_k <= w->experts, "moe: top_k must be within 1..16 and <= experts");
    STRIX_REQUIRE(static_cast<uint64_t>(rows) * w->top_k < (1ULL << 31), "moe: too many assignments");
    // rows are one grid dimension of the prologue and of the merge: every entry refuses a larger batch before its first launch
    STRIX_REQUIRE(rows <= 65535U, "moe: at most 65535 rows per call");
    // plan items are one grid dimension of the expert launches
    STRIX_REQUIRE(cls != kIntegerClass || item_bound(*w, rows) <= 65535U, "moe: too many work items for one call (experts + rows * top_k / 4 must stay below 65536)");
    wv = *w;
    if (wv.gate_row_stride == 0) wv.gate_row_stride = moe_row_bytes(w->gate_type, w->hidden);
    if (wv.gate_expert_stride == 0) wv.gate_expert_stride = wv.gate_row_stride * w->ffn;
    if (wv.down_row_stride == 0) wv.down_row_stride = moe_row_bytes(w->down_type, w->ffn);
    if (wv.down_expert_stride == 0) wv.down_expert_stride = wv.down_row_stride * w->hidden;
    const uint32_t down_unit = w->down_type == MI355_TYPE_Q6_K ? 2U : 16U;        // Q6_K blocks are 210 bytes
    STRIX_REQUIRE(wv.gate_row_stride % 16U == 0 && wv.gate_expert_stride % 16U == 0 && wv.down_row_stride % down_unit == 0 &&
                  wv.down_expert_stride % down_unit == 0, "moe: weight strides must be multiples of 16 bytes (Q6_K down: 2)");
    STRIX_REQUIRE(wv.gate_row_stride < (1ULL << 27) && wv.down_row_stride < (1ULL << 27), "moe: weight row stride must be below 128 MiB");
    STRIX_REQUIRE(wv.gate_row_stride >= moe_row_bytes(w->gate_type, w->hidden) &&
                  wv.down_row_stride >= moe_row_bytes(w->down_type, w->ffn), "moe: weight row stride shorter than the row");
    // (a stage that reads no weights is admitted on the geometry alone)
    STRIX_REQUIRE(!need_tensors || (w->gate && w->up && w->down && aligned(w->gate, 16) && aligned(w->up, 16) && aligned(w->down, 16)),
                  "moe: weight pointers must be non-null and 16-byte aligned");
    STRIX_REQUIRE(w->exp_kind <= MI355_EXP_DECLARED, "moe: unknown exp kind");
    // the clamp trait: +infinity (or the zero-initialised 0) = none, else finite and positive (src/moe_a8_down_contract.cpp:57)
    if (wv.swiglu_limit == 0.0F) wv.swiglu_limit = INFINITY;
    STRIX_REQUIRE(wv.swiglu_limit > 0.0F, "moe: swiglu_limit must be +infinity (none) or finite and positive");
    STRIX_REQUIRE(r->routes && r->route_weights && r->codes && r->deltas && r->sums && r->status && r->down_codes && r->down_deltas &&
                  r->down_sums && r->rawdots && r->output && r->plan && r->job_status, "moe: a required row view is null");
    STRIX_REQUIRE(aligned(r->codes, 16) && aligned(r->down_codes, 16) && aligned(r->plan, 16) && aligned(r->rawdots, 16) &&
                  aligned(r->deltas, 4) && aligned(r->down_deltas, 4), "moe: row views must be 16-byte aligned");
    STRIX_REQUIRE(r->output_stride >= w->hidden, "moe: output stride shorter than hidden");
    return MI355_OK;
}

}  // namespace strix950

// ============================================================================================================ C ABI
using namespace strix950;

extern "C" {

const char* mi355_last_error(void) { return g_error.c_str(); }
const char* mi355_version(void) { return "mi355-strix 0.1 (gfx950)"; }

const char* mi355_numerical_identity(uint32_t weight_type, int down) {
    // Identity strings are the admission tokens of the reference's contracts (include/strix/moe_q4k_a8_contract.hpp:24-29,
    // include/strix/moe_a8_down_contract.hpp:9-28); a caller hands over the token of the arithmetic it approved. The tokens are
    // returned verbatim because the bits are the same: "wave32" in the probe tokens names the reference's reduction tree
    // (pairs ascending, four super-block partials folded by a two-level tree), which the 64-lane kernels here reproduce.
    if (!down) {
        if (weight_type == MI355_TYPE_Q4_K)
            return "strix-moe-q4k-a8g32-probe-v2:f32-div-rne:g32-sym127-zero1-finite-noflush:"
                   "dot-s8xu8-i32:combine-separate-f32:pair-ascending-sb-tree4:writer-c0:wave32:proj-nonfinite=propagate-unqualified";
        if (weight_type == MI355_TYPE_Q5_K)
            return "strix-moe-q5k-a8g32-probe-v1:f32-div-rne:g32-sym127-zero1-finite-noflush:"
                   "dot-s8xu5qh-i32:combine-separate-f32:pair-ascending-sb-tree4:writer-c0:wave32:proj-nonfinite=propagate-unqualified";
        if (weight_type == MI355_TYPE_Q8_0) return "cpu-q8a8-tree32@1";
        return "";
    }
    if (weight_type == MI355_TYPE_Q4_K)
        return "q4k-a8g32-down-v1:s8xu4-i32:delta*((d*(sc*I))-(dmin*(m*S))):pair-ascending-sb-tree4:"
               "silu-div-expf-times-up:g32-sym127-f32delta-rne:tiny-lt2^-119-zero1:raw-slot-major:finite-failclosed";
    if (weight_type == MI355_TYPE_Q6_K)
        return "q6k-a8g32-down-v1:s8xs8-i32:delta*(d*(s0*I0+s1*I1)):pair-ascending-sb-tree4:"
               "silu-div-expf-times-up:g32-sym127-f32delta-rne:tiny-lt2^-119-zero1:raw-slot-major:finite-failclosed";
    if (weight_type == MI355_TYPE_Q5_1)
        return "q51-a8g32-down-v1:s8xu5-i32:delta*(d*S+m*C):separate-f32:"
               "silu-div-expf-times-up:g32-sym127-f32delta-rne:tiny-lt2^-119-zero1:"
               "blocks-mod4-ascending:tree-xor1-xor2:raw-slot-major:finite-failclosed";
    if (weight_type == MI355_TYPE_Q8_0)
        return "q80-a8g32-down-v1:s8xs8-i32:delta*(d*S):separate-f32:"
               "silu-div-expf-times-up:g32-sym127-f32delta-rne:tiny-lt2^-119-zero1:"
               "blocks-mod4-ascending:tree-xor1-xor2:raw-slot-major:finite-failclosed";
    return "";
}

int32_t mi355_dequantize_rows(uint32_t type, const void* rows, uint64_t row_stride, uint32_t n_rows, uint32_t elements,
                              float* out, uint64_t out_stride, mi355_stream stream) {
    if (type != MI355_TYPE_Q8_0 && type != MI355_TYPE_Q4_K) return fail(MI355_E_UNSUPPORTED, "dequantize: type must be Q8_0 (8) or Q4_K (12)");
    const uint32_t be = type == MI355_TYPE_Q8_0 ? 32U : 256U, bb = type == MI355_TYPE_Q8_0 ? kQ80Block : kQ4kBlock;
    STRIX_REQUIRE(rows && out, "dequantize: null pointer");
    STRIX_REQUIRE(elements % be == 0, "dequantize: row length is not a multiple of the block");
    STRIX_REQUIRE(row_stride >= static_cast<uint64_t>(elements / be) * bb && out_stride >= elements, "dequantize: stride shorter than the row");
    if (n_rows == 0 || elements == 0) return MI355_OK;
    const uint32_t gx = (elements + 255U) / 256U;
    for (uint32_t r0 = 0; r0 < n_rows; r0 += 65535U) {
        const uint32_t nr = n_rows - r0 < 65535U ? n_rows - r0 : 65535U;
        dequantize_rows_kernel<<<dim3(gx < 64U ? gx : 64U, nr), 256, 0, hs(stream)>>>(
            type, static_cast<const uint8_t*>(rows) + r0 * row_stride, row_stride, elements, out + r0 * out_stride, out_stride);
    }
    STRIX_LAUNCHED("dequantize_rows");
    return MI355_OK;
}

int32_t mi355_quantize_weight_rows(uint32_t type, const float* x, uint32_t n_rows, uint32_t elements, void* out, mi355_stream stream) {
    if (type != MI355_TYPE_Q8_0 && type != MI355_TYPE_Q4_K) return fail(MI355_E_UNSUPPORTED, "quantize_weight: type must be Q8_0 (8) or Q4_K (12)");
    const uint32_t be = type == MI355_TYPE_Q8_0 ? 32U : 256U;
    STRIX_REQUIRE(x && out, "quantize_weight: null pointer");
    STRIX_REQUIRE(elements % be == 0, "quantize_weight: row length is not a multiple of the block");
    const uint64_t blocks = static_cast<uint64_t>(n_rows) * (elements / be);
    if (blocks == 0) return MI355_OK;
    if (type == MI355_TYPE_Q8_0) {
        const uint64_t g = (blocks + 255U) / 256U;
        quantize_q8_0_rows_kernel<<<static_cast<uint32_t>(g < 65535U ? g : 65535U), 256, 0, hs(stream)>>>(x, blocks, static_cast<uint8_t*>(out));
    } else {
        const uint64_t g = (blocks + 63U) / 64U;
        quantize_q4_k_rows_kernel<<<static_cast<uint32_t>(g < 262144U ? g : 262144U), 64, 0, hs(stream)>>>(x, blocks, static_cast<uint8_t*>(out));
    }
    STRIX_LAUNCHED("quantize_weight_rows");
    return MI355_OK;
}

int32_t mi355_quantize_a8(const void* x, uint32_t kind, uint32_t rows, uint32_t width, uint64_t x_stride, int8_t* codes, float* deltas,
                          int32_t* sums, uint32_t* status, mi355_stream stream) {
    STRIX_REQUIRE(width % 32U == 0, "A8 activation width must be a multiple of 32");
    STRIX_REQUIRE(kind <= MI355_INPUT_BF16, "A8: unknown input kind");
    if (rows == 0 || width == 0) return MI355_OK;
    STRIX_REQUIRE(x && codes && deltas, "A8: null pointer");
    STRIX_REQUIRE(rows <= 65535U, "A8: at most 65535 rows per call");
    const dim3 grid((width / 32U + 7U) / 8U, rows);
    const uint8_t* xb = static_cast<const uint8_t*>(x);
    if (kind == MI355_INPUT_F32) quantize_a8_kernel<0><<<grid, 256, 0, hs(stream)>>>(xb, x_stride, width, codes, deltas, sums, status);
    else if (kind == MI355_INPUT_F16) quantize_a8_kernel<1><<<grid, 256, 0, hs(stream)>>>(xb, x_stride, width, codes, deltas, sums, status);
    else quantize_a8_kernel<2><<<grid, 256, 0, hs(stream)>>>(xb, x_stride, width, codes, deltas, sums, status);
    STRIX_LAUNCHED("quantize_a8");
    return MI355_OK;
}

int32_t mi355_dense_a8_quantize(const void* x, uint32_t kind, uint32_t rows, uint32_t width, uint64_t x_stride, int8_t* codes, float* deltas,
                                mi355_stream stream) {
    STRIX_REQUIRE(width % 32U == 0, "dense A8 activation width must be a multiple of 32");
    STRIX_REQUIRE(kind <= MI355_INPUT_BF16, "dense A8: unknown input kind");
    if (rows == 0 || width == 0) return MI355_OK;
    STRIX_REQUIRE(x && codes && deltas, "dense A8: null pointer");
    STRIX_REQUIRE(rows <= 65535U, "dense A8: at most 65535 rows per call");
    const dim3 grid((width / 32U + 7U) / 8U, rows);
    const uint8_t* xb = static_cast<const uint8_t*>(x);
    if (kind == MI355_INPUT_F32) quantize_a8_kernel<0><<<grid, 256, 0, hs(stream)>>>(xb, x_stride, width, codes, deltas, nullptr, nullptr, 1U);
    else if (kind == MI355_INPUT_F16) quantize_a8_kernel<1><<<grid, 256, 0, hs(stream)>>>(xb, x_stride, width, codes, deltas, nullptr, nullptr, 1U);
    else quantize_a8_kernel<2><<<grid, 256, 0, hs(stream)>>>(xb, x_stride, width, codes, deltas, nullptr, nullptr, 1U);
    STRIX_LAUNCHED("dense A8 quantize");
    return MI355_OK;
}

int32_t mi355_gemv_q8_0_a8_chain(const mi355_q8a8_view* v, mi355_stream stream) {
    STRIX_REQUIRE(v, "Q8_0 chain product: null view");
    STRIX_REQUIRE(v->in % 64U == 0 && v->in <= 32U * kGemvChainMaxGroups, "Q8_0 chain product: width must be a multiple of 64, at most 8192");   // dense_a8_width, src/hip_q8_rows_gemv.hpp:1184
    STRIX_REQUIRE(!v->accumulate, "Q8_0 chain product: the chain starts at +0 (no accumulate)");
    if (v->rows == 0 || v->count == 0) return MI355_OK;
    STRIX_REQUIRE(v->weight && v->codes && v->deltas && v->out, "Q8_0 chain product: null pointer");
    STRIX_REQUIRE(aligned(v->weight, 4) && v->row_bytes % 4U == 0, "Q8_0 chain product: weight rows must be 4-byte aligned");
    STRIX_REQUIRE(aligned(v->codes, 16) && v->x_stride % 32U == 0 && v->x_stride >= v->in, "Q8_0 chain product: codes must be 16-byte aligned with x_stride a multiple of 32");
    STRIX_REQUIRE(v->row_bytes >= v->in / 32U * kQ80Block && v->out_stride >= v->count && v->rows <= 65535U, "Q8_0 chain product: stride shorter than the row, or too many rows");
    gemv_q8_0_a8_kernel<1, true, true><<<dim3((v->count + 7U) / 8U, v->rows), 256, 0, hs(stream)>>>(*v);
    STRIX_LAUNCHED("gemv_q8_0_a8 chain");
    return MI355_OK;
}

int32_t mi355_rmsnorm_f32(const float* x, const float* w, uint32_t n, float eps, float* y, uint32_t rows, mi355_stream stream) {
    if (rows == 0 || n == 0) return MI355_OK;
    STRIX_REQUIRE(x && y, "rmsnorm: null pointer");
    STRIX_REQUIRE(rows <= 0x7fffffffU, "rmsnorm: too many rows");
    rmsnorm_f32_kernel<<<rows, n >= 512U ? 256 : 128, 0, hs(stream)>>>(x, w, n, eps, y);
    STRIX_LAUNCHED("rmsnorm_f32");
    return MI355_OK;
}

int32_t mi355_gemv_q8_0_a8(const mi355_q8a8_view* v, mi355_stream stream) {
    STRIX_REQUIRE(v, "Q8_0 product: null view");
    STRIX_REQUIRE(v->in % 32U == 0, "Q8_0 product width must be a multiple of 32");
    if (v->rows == 0 || v->count == 0) return MI355_OK;
    STRIX_REQUIRE(v->weight && v->codes && v->deltas && v->out, "Q8_0 product: null pointer");
    STRIX_REQUIRE(aligned(v->weight, 2) && v->row_bytes % 2U == 0, "Q8_0 product: weight rows must be 2-byte aligned");
    STRIX_REQUIRE(aligned(v->codes, 16) && v->x_stride % 32U == 0 && v->x_stride >= v->in, "Q8_0 product: codes must be 16-byte aligned with x_stride a multiple of 32");
    STRIX_REQUIRE(v->row_bytes >= v->in / 32U * kQ80Block && v->out_stride >= v->count, "Q8_0 product: stride shorter than the row");
    const uint32_t grid = (v->count + 7U) / 8U;
    const bool dw = aligned(v->weight, 4) && v->row_bytes % 4U == 0;
    hipStream_t st = hs(stream);
    // up to RB activation rows share one sweep of a weight row; more rows are further blocks of the same launch (grid.y)
    const auto launch = [&](auto rb_constant) {
        constexpr int RB = decltype(rb_constant)::value;
        const dim3 g(grid, (v->rows + RB - 1U) / RB);
        if (dw) gemv_q8_0_a8_kernel<RB, true><<<g, 256, 0, st>>>(*v);
        else gemv_q8_0_a8_kernel<RB, false><<<g, 256, 0, st>>>(*v);
    };
    STRIX_REQUIRE((v->rows + 15U) / 16U <= 65535U, "Q8_0 product: too many rows for one launch");
    if (v->rows == 1U) launch(std::integral_constant<int, 1>{});
    else if (v->rows == 2U) launch(std::integral_constant<int, 2>{});
    else if (v->rows <= 4U) launch(std::integral_constant<int, 4>{});
    else if (v->rows <= 8U) launch(std::integral_constant<int, 8>{});
    else launch(std::integral_constant<int, 16>{});            // (32 rows per sweep measured slower: 5.0 vs 4.05 ms on 4096 rows)
    STRIX_LAUNCHED("gemv_q8_0_a8");
    return MI355_OK;
}

namespace {
int32_t check_route(const mi355_route_policy* p, const void* x, uint32_t kind, uint32_t hidden, uint64_t x_stride, const float* wr,
                    const uint32_t* ids, const float* weights, const float* scores) {
    STRIX_REQUIRE(p && x && wr && ids && weights && scores, "route: null pointer");
    STRIX_REQUIRE(p->experts > 0 && p->experts <= kRouteMaxExperts && p->top_k > 0 && p->top_k <= kRouteMaxTopK && p->top_k <= p->experts,
                  "route policy: need 0 < top_k <= experts, experts <= 1024, top_k <= 16");
    STRIX_REQUIRE(p->shared_experts <= 4U && p->top_k + p->shared_experts <= kRouteMaxTopK && p->experts + p->shared_experts <= kRouteMaxExperts,
                  "route policy: at most 4 always-on experts, top_k + shared <= 16, experts + shared <= 1024");
    STRIX_REQUIRE(hidden > 0 && hidden <= kRouteMaxHidden && hidden % 32U == 0, "route: hidden must be a multiple of 32 within 16384");
    STRIX_REQUIRE(kind <= MI355_INPUT_BF16 && p->logits_order <= MI355_LOGITS_LANE32_BUTTERFLY, "route: unknown input kind or logits order");
    STRIX_REQUIRE(p->exp_kind <= MI355_EXP_LIBM, "route policy: unknown exp kind");
    STRIX_REQUIRE(aligned(wr, 16) && aligned(x, 16) && x_stride % 16U == 0, "route: router weight, activations and their row stride must be 16-byte aligned");
    return MI355_OK;
}
// Logits of every (row, expert) into a.scores. Decode batches: one block per (row, 8 experts), plus a.quant_blocks blocks
// in the fused form; larger batches: one block per (8 rows, 8 experts).
void launch_route_logits(RouteArgs& a, hipStream_t st) {
    const uint32_t neb = (a.p.experts + 7U) / 8U;
    if (a.rows <= kFusedMaxRows) {
        a.route_blocks = neb * a.rows;
        const uint32_t blocks = a.route_blocks + a.quant_blocks;
        if (a.norm_on) {
            if (a.kind == MI355_INPUT_F32) route_decode_kernel<0, true><<<blocks, 64, 0, st>>>(a);
            else if (a.kind == MI355_INPUT_F16) route_decode_kernel<1, true><<<blocks, 64, 0, st>>>(a);
            else route_decode_kernel<2, true><<<blocks, 64, 0, st>>>(a);
        } else if (a.kind == MI355_INPUT_F32) route_decode_kernel<0><<<blocks, 64, 0, st>>>(a);
        else if (a.kind == MI355_INPUT_F16) route_decode_kernel<1><<<blocks, 64, 0, st>>>(a);
        else route_decode_kernel<2><<<blocks, 64, 0, st>>>(a);
    } else if (a.p.logits_order == MI355_LOGITS_FMA_ASCENDING && (a.rows + kBatchTile - 1U) / kBatchTile <= 65535U) {
        const dim3 grid((a.p.experts + kBatchTile - 1U) / kBatchTile, (a.rows + kBatchTile - 1U) / kBatchTile);
        if (a.kind == MI355_INPUT_F32) route_batch_kernel<0><<<grid, 256, 0, st>>>(a);
        else if (a.kind == MI355_INPUT_F16) route_batch_kernel<1><<<grid, 256, 0, st>>>(a);
        else route_batch_kernel<2><<<grid, 256, 0, st>>>(a);
    } else {
        a.route_blocks = neb * ((a.rows + 7U) / 8U);
        if (a.kind == MI355_INPUT_F32) route_logits_kernel<0><<<a.route_blocks, 64, 0, st>>>(a);
        else if (a.kind == MI355_INPUT_F16) route_logits_kernel<1><<<a.route_blocks, 64, 0, st>>>(a);
        else route_logits_kernel<2><<<a.route_blocks, 64, 0, st>>>(a);
    }
}
}  // namespace

int32_t mi355_moe_route(const mi355_route_policy* p, const void* x, uint32_t kind, uint32_t rows, uint32_t hidden, uint64_t x_stride,
                        const float* wr, const float* bias, uint32_t* ids, float* weights, float* scores, mi355_stream stream) {
    if (const int32_t rc = check_route(p, x, kind, hidden, x_stride, wr, ids, weights, scores)) return rc;
    if (rows == 0) return MI355_OK;
    RouteArgs a{};
    a.p = *p; a.x = static_cast<const uint8_t*>(x); a.kind = kind; a.x_stride = x_stride; a.rows = rows; a.hidden = hidden;
    a.wr = wr; a.bias = bias; a.ids = ids; a.weights = weights; a.scores = scores;
    launch_route_logits(a, hs(stream));
    route_select_kernel<<<rows, 64, 0, hs(stream)>>>(a);
    STRIX_LAUNCHED("moe_route");
    return MI355_OK;
}

size_t mi355_moe_prefill_f16_workspace_bytes(uint32_t hidden, uint32_t ffn, uint32_t rows, uint32_t top_k) {
    return pf_workspace_bytes(hidden, ffn, rows, top_k);
}

size_t mi355_moe_plan_words(uint32_t experts, uint32_t rows, uint32_t top_k) {
    return plan_words_total(experts, rows * top_k);
}

int32_t mi355_moe_enqueue_prologue(const mi355_moe_weights* w, const mi355_moe_rows* r, uint32_t rows, mi355_stream stream) {
    mi355_moe_weights wv;
    if (const int32_t rc = check_moe(w, r, rows, wv)) return rc;
    STRIX_REQUIRE(r->input && r->input_kind <= MI355_INPUT_BF16, "moe prologue: input view invalid");
    clear_validate_kernel<<<rows, 64, 0, hs(stream)>>>(r->routes, r->route_weights, wv.experts, wv.top_k, r->status, r->job_status);
    STRIX_LAUNCHED("moe clear/validate");
    return mi355_quantize_a8(r->input, r->input_kind, rows, wv.hidden, r->input_stride, r->codes, r->deltas, r->sums, r->status, stream);
}

int32_t mi355_moe_enqueue_csr(const mi355_moe_weights* w, const mi355_moe_rows* r, uint32_t rows, mi355_stream stream) {
    mi355_moe_weights wv;
    if (const int32_t rc = check_moe(w, r, rows, wv)) return rc;
    launch_plan(dense_routes(r->routes, wv.top_k), wv.experts, rows * wv.top_k, plan_split(wv, rows), item_bound(wv, rows), r->plan, hs(stream));
    STRIX_LAUNCHED("moe plan");
    return MI355_OK;
}

int32_t mi355_moe_enqueue_project(const mi355_moe_weights* w, const mi355_moe_rows* r, uint32_t rows, mi355_stream stream) {
    mi355_moe_weights wv;
    if (const int32_t rc = check_moe(w, r, rows, wv)) return rc;
    launch_project(wv, rows_k(*r, wv), rows, item_bound(wv, rows), hs(stream));
    STRIX_LAUNCHED("moe project");
    return MI355_OK;
}

int32_t mi355_moe_enqueue_down(const mi355_moe_weights* w, const mi355_moe_rows* r, uint32_t rows, mi355_stream stream) {
    mi355_moe_weights wv;
    if (const int32_t rc = check_moe(w, r, rows, wv)) return rc;
    launch_down(wv, rows_k(*r, wv), rows, item_bound(wv, rows), hs(stream));
    STRIX_LAUNCHED("moe down");
    return MI355_OK;
}

}  // extern "C"
namespace {
// shared_slots: the last slots of every row are always-on experts (a layer call with policy->shared_experts)
int32_t enqueue_merge(const mi355_moe_weights* w, const mi355_moe_rows* r, uint32_t rows, uint32_t form, mi355_stream stream, uint32_t shared_slots) {
    mi355_moe_weights wv;
    if (const int32_t rc = check_moe(w, r, rows, wv, kAnyClass)) return rc;
    STRIX_REQUIRE(form <= MI355_COMBINE_MULADD_ASCENDING_EXPERT, "moe merge: unknown combine form");
    STRIX_REQUIRE(rows <= 65535U, "moe merge: at most 65535 rows per call");
    RowsK k = rows_k(*r, wv);
    k.shared_slots = shared_slots;
    // four columns per thread once that still leaves every compute unit several workgroups (4096 rows x 4096: 194 -> 113 us;
    // a decode batch is faster with one column per thread: 16 rows x 6144: 8.5 against 10.9 us)
    const bool quads = static_cast<uint64_t>(rows) * ((wv.hidden + 1023U) / 1024U) >= 4ULL * compute_units() && wv.hidden % 4U == 0 && aligned(k.rawdots, 16) && k.rawdots_rs % 16U == 0 && aligned(k.output, 16) && k.output_stride % 4U == 0 &&
                       (!k.base || (aligned(k.base, 16) && k.base_rs % 16U == 0));
    if (quads) merge_kernel<4><<<dim3((wv.hidden + 1023U) / 1024U, rows), 256, 0, hs(stream)>>>(wv, k, form);
    else merge_kernel<1><<<dim3((wv.hidden + 255U) / 256U, rows), 256, 0, hs(stream)>>>(wv, k, form);
    STRIX_LAUNCHED("moe merge");
    return MI355_OK;
}
}  // namespace
extern "C" {

int32_t mi355_moe_enqueue_merge(const mi355_moe_weights* w, const mi355_moe_rows* r, uint32_t rows, uint32_t form, mi355_stream stream) {
    return enqueue_merge(w, r, rows, form, stream, 0U);
}

int32_t mi355_moe_enqueue(const mi355_moe_weights* w, const mi355_moe_rows* r, uint32_t rows, uint32_t form, mi355_stream stream) {
    mi355_moe_weights wv;
    if (const int32_t rc = check_moe(w, r, rows, wv)) return rc;   // the whole bundle is validated before the first enqueue
    STRIX_REQUIRE(form <= MI355_COMBINE_MULADD_ASCENDING_EXPERT, "moe: unknown combine form");
    STRIX_REQUIRE(r->input && r->input_kind <= MI355_INPUT_BF16, "moe: input view invalid");
    if (const int32_t rc = mi355_moe_enqueue_prologue(w, r, rows, stream)) return rc;
    // a dense matrix on the pair-per-lane sweep reads no expert plan
    if (!(dense_pairs_ok(wv, rows) && r->gate_out && r->up_out))
        if (const int32_t rc = mi355_moe_enqueue_csr(w, r, rows, stream)) return rc;
    if (const int32_t rc = mi355_moe_enqueue_project(w, r, rows, stream)) return rc;
    // a dense top-1 job: the down launch publishes each row's output with its one unweighted value (no merge launch)
    RowsK k = rows_k(*r, wv);
    if (wv.experts == 1U && wv.top_k == 1U && rows <= 65535U) k.top1_form = form + 1U;
    const bool published = launch_down(wv, k, rows, item_bound(wv, rows), hs(stream));
    STRIX_LAUNCHED("moe down");
    if (published) return MI355_OK;
    return mi355_moe_enqueue_merge(w, r, rows, form, stream);
}

}  // extern "C"

namespace {
// mi355_moe_enqueue by halves: front = prologue, plan, gate / up; back = down rows, combine.
int32_t enqueue_staged(const mi355_moe_weights* w, const mi355_moe_rows* r, uint32_t rows, uint32_t form, mi355_stream stream, bool do_front, bool do_back,
                       uint32_t shared_slots = 0) {
    mi355_moe_weights wv;
    if (const int32_t rc = check_moe(w, r, rows, wv)) return rc;
    STRIX_REQUIRE(form <= MI355_COMBINE_MULADD_ASCENDING_EXPERT, "moe: unknown combine form");
    if (do_front) {
        STRIX_REQUIRE(r->input && r->input_kind <= MI355_INPUT_BF16, "moe: input view invalid");
        if (const int32_t rc = mi355_moe_enqueue_prologue(w, r, rows, stream)) return rc;
        if (!(dense_pairs_ok(wv, rows) && r->gate_out && r->up_out))
            if (const int32_t rc = mi355_moe_enqueue_csr(w, r, rows, stream)) return rc;
        if (const int32_t rc = mi355_moe_enqueue_project(w, r, rows, stream)) return rc;
    }
    if (!do_back) return MI355_OK;
    RowsK k = rows_k(*r, wv);
    if (wv.experts == 1U && wv.top_k == 1U && rows <= 65535U) k.top1_form = form + 1U;
    const bool published = launch_down(wv, k, rows, item_bound(wv, rows), hs(stream));
    STRIX_LAUNCHED("moe down");
    if (published) return MI355_OK;
    return enqueue_merge(w, r, rows, form, stream, shared_slots);
}

// RMSNorm of rows of any input kind into fp32 rows (the staged form of the fused norm): rmsnorm_f32_kernel's order.
template <int KIND>
__global__ __launch_bounds__(64) void rmsnorm_rows_kernel(const uint8_t* x, uint64_t x_stride, const float* w, uint32_t n, float eps, float* y) {
    __shared__ float partial[256];
    const uint8_t* xr = x + blockIdx.x * x_stride;
    const float r = row_norm_factor<KIND>(partial, xr, n, eps);
    float* yr = y + static_cast<size_t>(blockIdx.x) * n;
    for (uint32_t i = threadIdx.x; i < n; i += 64U) {
        const float v = load_activation<KIND>(xr, i) * r;
        yr[i] = w ? v * w[i] : v;
    }
}

struct LayerNorm { bool on; const float* weight; float eps; float* normed; };
std::atomic<uint32_t> g_early_perturb{0};
std::atomic<bool> g_down_merge_flat{true};

// phase: 0 = the whole layer; 1 = its front half (router, A8 prologue, plan, gate / up); 2 = its back half (down rows, combine) on
// what a front call with the same arguments left in the row views.
enum { kLayerWhole = 0, kLayerFront = 1, kLayerBack = 2 };
// down rows + combine of a decode batch whose every workgroup is resident: dense rows of at most four super-blocks stream as
// contiguous stages (down_merge_flat_kernel), other shapes as 144-byte blocks of 64 rows (down_merge_kernel)
void launch_down_merge(const mi355_moe_weights& wv, const RowsK& k, uint32_t rows, uint32_t items, uint32_t form, hipStream_t st) {
    const dim3 grid(wv.hidden / 64U, rows);
    const uint32_t threads = 64U * wv.top_k, B = wv.ffn / 256U;
    const bool flat = wv.down_row_stride == static_cast<uint64_t>(B) * kQ4kBlock && wv.down_expert_stride % 16U == 0 && !k.h.table && k.h.codes &&
                      aligned(k.h.codes, 16) && aligned(k.h.deltas, 16) && aligned(k.h.sums, 16) && wv.ffn % 256U == 0 && g_down_merge_flat.load(std::memory_order_relaxed);
    if (flat && B == 1U) down_merge_flat_kernel<1><<<grid, threads, 0, st>>>(wv, k, items, form);
    else if (flat && B == 2U) down_merge_flat_kernel<2><<<grid, threads, 0, st>>>(wv, k, items, form);
    else if (flat && B == 3U) down_merge_flat_kernel<3><<<grid, threads, 0, st>>>(wv, k, items, form);
    else if (flat && B == 4U) down_merge_flat_kernel<4><<<grid, threads, 0, st>>>(wv, k, items, form);
    else down_merge_kernel<<<grid, threads, 0, st>>>(wv, k, items, form);
}

int32_t enqueue_layer(const mi355_route_policy* p, const float* router_weight, const float* logit_bias, float* scores, const LayerNorm& norm,
                      const mi355_moe_weights* w, const mi355_moe_rows* r, uint32_t rows, uint32_t form, mi355_stream stream, uint32_t phase = kLayerWhole) {
    const bool do_front = phase != kLayerBack, do_back = phase != kLayerFront;
    mi355_moe_weights wv;
    if (const int32_t rc = check_moe(w, r, rows, wv)) return rc;
    const auto layer_rows = [&] { RowsK k = rows_k(*r, wv); k.shared_slots = p->shared_experts; return k; };
    STRIX_REQUIRE(form <= MI355_COMBINE_MULADD_ASCENDING_EXPERT, "moe: unknown combine form");
    STRIX_REQUIRE(r->input && r->input_kind <= MI355_INPUT_BF16, "moe: input view invalid");
    uint32_t* ids = const_cast<uint32_t*>(r->routes);
    float* weights = const_cast<float*>(r->route_weights);
    if (const int32_t rc = check_route(p, r->input, r->input_kind, wv.hidden, r->input_stride, router_weight, ids, weights, scores)) return rc;
    STRIX_REQUIRE(p->experts + p->shared_experts == wv.experts && p->top_k + p->shared_experts == wv.top_k,
                  "moe layer: router policy (experts, top_k, always-on experts) and expert tensors disagree on experts / top_k");
    STRIX_REQUIRE(!norm.on || (norm.normed && aligned(norm.normed, 16) && (!norm.weight || aligned(norm.weight, 16)) && norm.eps >= 0.0F),
                  "moe layer: the fused RMSNorm needs a 16-byte aligned fp32 [rows][hidden] view for the normalised rows, aligned weights, eps >= 0");
    hipStream_t st = hs(stream);
    if (rows > kFusedMaxRows || plan_split(wv, rows) != 1U) {      // large batches, and decode batches over large experts (shared sweeps): router, then the staged prologue / plan
        mi355_moe_rows staged = *r;
        if (norm.on && do_front) {
            const uint8_t* x = static_cast<const uint8_t*>(r->input);
            if (r->input_kind == MI355_INPUT_F32) rmsnorm_rows_kernel<0><<<rows, 64, 0, st>>>(x, r->input_stride, norm.weight, wv.hidden, norm.eps, norm.normed);
            else if (r->input_kind == MI355_INPUT_F16) rmsnorm_rows_kernel<1><<<rows, 64, 0, st>>>(x, r->input_stride, norm.weight, wv.hidden, norm.eps, norm.normed);
            else rmsnorm_rows_kernel<2><<<rows, 64, 0, st>>>(x, r->input_stride, norm.weight, wv.hidden, norm.eps, norm.normed);
            STRIX_LAUNCHED("moe layer norm");
        }
        if (norm.on) { staged.input = norm.normed; staged.input_kind = MI355_INPUT_F32; staged.input_stride = 4ULL * wv.hidden; }
        if (do_front)
            if (const int32_t rc = mi355_moe_route(p, staged.input, staged.input_kind, rows, wv.hidden, staged.input_stride, router_weight, logit_bias, ids, weights, scores, stream)) return rc;
        return enqueue_staged(w, &staged, rows, form, stream, do_front, do_back, p->shared_experts);
    }
    RouteArgs a{};
    a.p = *p; a.x = static_cast<const uint8_t*>(r->input); a.kind = r->input_kind; a.x_stride = r->input_stride; a.rows = rows; a.hidden = wv.hidden;
    a.wr = router_weight; a.bias = logit_bias; a.ids = ids; a.weights = weights; a.scores = scores;
    a.codes = r->codes; a.deltas = r->deltas; a.sums = r->sums; a.status = r->status; a.job_status = r->job_status; a.plan = r->plan;
    a.quant_blocks = (rows * (wv.hidden / 32U) + 7U) / 8U;
    a.norm_on = norm.on ? 1U : 0U; a.norm_w = norm.weight; a.norm_eps = norm.eps; a.normed = norm.normed;
    const uint32_t items = rows * wv.top_k;
    // Early routes (route_early.hpp): the expert choice from lane-parallel logits in a short first launch, the exact router beside
    // the projection, down rows + combine on the verified work items. Taken where the 64-row projection sweep and the down +
    // combine launch serve the batch.
    // Up to two rounds of the down + combine launch's workgroups (each fills a compute unit's LDS): at hidden 2048 / ffn 768, 9..16
    // rows take 61.5 / 63.2 / 71.4 / 78.0 us (9, 10, 12, 16 rows) against 66.8 / 75.4 / 88.4 / 100 us on the router launch, the
    // 64-row projection and the staged down rows + combine.
    // From 8 assignments on (one row of top-8): measured at hidden 2048 / ffn 768 against the three launches of the smallest batches
    // (router, 16-row projection, 16-row down + combine): 1 row 28.7 / 31.3 us, 2 rows 31.6 / 35.4, 3 rows 33.4 / 37.8, 4 rows
    // 35.7 / 40.3, 5 rows 38.4 / 48.6, 6 rows 41.2 / 57.8.
    if (!norm.on && p->shared_experts == 0 && p->logits_order == MI355_LOGITS_FMA_ASCENDING && wv.gate_type == MI355_TYPE_Q4_K &&
        wv.down_type == MI355_TYPE_Q4_K && items >= kEarlyMinAssignments && wv.experts > 1U && wv.top_k <= kDownMergeSlots && items <= kEarlyMaxAssignments &&
        wv.hidden <= kSideMaxHidden && wv.hidden % 64U == 0 && (wv.hidden / 64U) * rows <= 2U * compute_units() && 2U * wv.experts <= wv.top_k * wv.hidden) {
        a.awords = r->plan + kPlanAwordsAt;
        a.early_perturb = g_early_perturb.load(std::memory_order_relaxed);
        // the early logits of row i (64-bit words) live in the row's (still unused) unweighted-output block: the exact logits own `scores`
        a.early_logits = r->rawdots; a.early_stride = wv.top_k * wv.hidden;
        RowsK k = layer_rows();
        k.awords = a.awords;
        RowsK front = k;
        front.plan = nullptr;              // (the front launch names its assignments itself: the work items are written inside it)
        const FrontBlocks nb{rows * ((p->experts + kEarlyExperts - 1U) / kEarlyExperts), a.quant_blocks, rows * ((p->experts + kSideExperts - 1U) / kSideExperts)};
        const uint32_t blocks = nb.early + nb.prologue + nb.side + items * (wv.ffn / 32U);
        if (do_front) {
            if (a.kind == MI355_INPUT_F32) layer_front_kernel<0><<<blocks, 64, 0, st>>>(wv, front, items, a, nb);
            else if (a.kind == MI355_INPUT_F16) layer_front_kernel<1><<<blocks, 64, 0, st>>>(wv, front, items, a, nb);
            else layer_front_kernel<2><<<blocks, 64, 0, st>>>(wv, front, items, a, nb);
            STRIX_LAUNCHED("moe layer early routes + gate / up");
        }
        if (do_back) {
            launch_down_merge(wv, k, rows, items, form, st);
            STRIX_LAUNCHED("moe layer experts + combine");
        }
        return MI355_OK;
    }
    if (do_front) {
        launch_route_logits(a, st);
        STRIX_LAUNCHED("moe layer router");
    }
    // the fused router planned one item per routed assignment (and one per four rows of an always-on expert)
    if (p->shared_experts) {       // items of several rows: the 64-row sweeps
        if (do_front) {
            launch_project(wv, layer_rows(), rows, items, st, true);
            STRIX_LAUNCHED("moe layer gate / up");
        }
        if (!do_back) return MI355_OK;
        launch_down(wv, layer_rows(), rows, items, st, true);
        STRIX_LAUNCHED("moe layer experts");
        return enqueue_merge(w, r, rows, form, stream, p->shared_experts);
    }
    if (do_front) launch_project(wv, layer_rows(), rows, items, st);
    if (!do_back) return MI355_OK;
    // down rows and the combine in one launch (the fused router's plan: one item per assignment, in assignment order).
    // A workgroup of that kernel fills a compute unit's LDS; up to four rounds of them it still beats the staged pair of launches
    // (hidden 3072 / ffn 768, 64 experts top-8: 8 rows 76.3 against 82.4 us, 16 rows 115.8 against 121.6 us)
    if (!quad_sweep(wv, rows) && wv.down_type == MI355_TYPE_Q4_K && wv.experts > 1U && wv.top_k <= kDownMergeSlots && wv.hidden % 64U == 0 &&
        (wv.hidden / 64U) * rows <= 4U * compute_units()) {
        launch_down_merge(wv, layer_rows(), rows, items, form, st);
        STRIX_LAUNCHED("moe layer experts + combine");
        return MI355_OK;
    }
    if (quad_sweep(wv, rows) && wv.down_type == MI355_TYPE_Q4_K && wv.top_k <= kDownMergeSlots && wv.hidden % kQuadRows == 0 && rows <= 65535U) {
        const dim3 grid(wv.hidden / kQuadRows, rows);
        if (rows <= 2U) down_merge_quad_kernel<4><<<grid, 64U * wv.top_k, 0, st>>>(wv, layer_rows(), items, form);
        else down_merge_quad_kernel<2><<<grid, 64U * wv.top_k, 0, st>>>(wv, layer_rows(), items, form);
        STRIX_LAUNCHED("moe layer experts + combine");
        return MI355_OK;
    }
    if (wv.down_type == MI355_TYPE_Q8_0 && wv.top_k <= kDownMergeSlots && wv.hidden % 16U == 0 && wv.ffn % 128U == 0 && rows <= 65535U) {
        down_merge_q8_0_kernel<<<dim3(wv.hidden / 16U, rows), 64U * wv.top_k, 0, st>>>(wv, layer_rows(), items, form);
        STRIX_LAUNCHED("moe layer experts + combine");
        return MI355_OK;
    }
    if (wv.down_type == MI355_TYPE_Q5_1 && wv.top_k <= kDownMergeSlots && wv.hidden % 16U == 0 && rows <= 65535U && wv.ffn % 256U == 0 &&
        wv.down_row_stride % 16U == 0 && wv.down_expert_stride % 16U == 0) {       // (what down_q51_ring_kernel's copies need)
        down_merge_q51_kernel<2><<<dim3(wv.hidden / 16U, rows), 64U * wv.top_k, 0, st>>>(wv, layer_rows(), items, form);
        STRIX_LAUNCHED("moe layer experts + combine");
        return MI355_OK;
    }
    if (wv.down_type == MI355_TYPE_Q6_K && wv.top_k <= kDownMergeSlots && wv.hidden % 16U == 0 && rows <= 65535U) {
        down_merge_q6k_kernel<<<dim3(wv.hidden / 16U, rows), 64U * wv.top_k, 0, st>>>(wv, layer_rows(), items, form);
        STRIX_LAUNCHED("moe layer experts + combine");
        return MI355_OK;
    }
    launch_down(wv, layer_rows(), rows, items, st);
    STRIX_LAUNCHED("moe layer experts");
    return enqueue_merge(w, r, rows, form, stream, p->shared_experts);
}
}  // namespace

extern "C" {

void mi355_debug_early_route_perturb(uint32_t amount) { g_early_perturb.store(amount, std::memory_order_relaxed); }
void mi355_debug_down_merge_flat(uint32_t on) { g_down_merge_flat.store(on != 0, std::memory_order_relaxed); }

int32_t mi355_moe_enqueue_layer(const mi355_route_policy* p, const float* router_weight, const float* logit_bias, float* scores,
                                const mi355_moe_weights* w, const mi355_moe_rows* r, uint32_t rows, uint32_t form, mi355_stream stream) {
    return enqueue_layer(p, router_weight, logit_bias, scores, LayerNorm{false, nullptr, 0.0F, nullptr}, w, r, rows, form, stream);
}

int32_t mi355_moe_enqueue_layer_front(const mi355_route_policy* p, const float* router_weight, const float* logit_bias, float* scores,
                                      const mi355_moe_weights* w, const mi355_moe_rows* r, uint32_t rows, uint32_t form, mi355_stream stream) {
    return enqueue_layer(p, router_weight, logit_bias, scores, LayerNorm{false, nullptr, 0.0F, nullptr}, w, r, rows, form, stream, kLayerFront);
}

int32_t mi355_moe_enqueue_layer_back(const mi355_route_policy* p, const float* router_weight, const float* logit_bias, float* scores,
                                     const mi355_moe_weights* w, const mi355_moe_rows* r, uint32_t rows, uint32_t form, mi355_stream stream) {
    return enqueue_layer(p, router_weight, logit_bias, scores, LayerNorm{false, nullptr, 0.0F, nullptr}, w, r, rows, form, stream, kLayerBack);
}

int32_t mi355_moe_enqueue_layer_normed(const mi355_route_policy* p, const float* router_weight, const float* logit_bias, float* scores,
                                       const float* norm_weight, float norm_eps, float* normed, const mi355_moe_weights* w, const mi355_moe_rows* r,
                                       uint32_t rows, uint32_t form, mi355_stream stream) {
    return enqueue_layer(p, router_weight, logit_bias, scores, LayerNorm{true, norm_weight, norm_eps, normed}, w, r, rows, form, stream);
}

}  // extern "C"
namespace {
// What the prefill kernels see of the caller's rows: dense bundles and the strided PrefillRows views fill it alike.
struct PrefillViews {
    const void* input; uint64_t input_stride;
    RoutesView routes;
    uint32_t* status; uint64_t status_rs;
    uint32_t* job_status;
    float* rawdots; uint64_t rawdots_rs;          // rawdots_rs == 0: dense [assignment][hidden]
    uint32_t rawdots_bf16;
    uint32_t* plan;
    void* h_f16;
};
// expert plan, sub-block sums of the input rows, gate / up + SwiGLU, down rows (the status words are already written)
int32_t enqueue_prefill_core(const mi355_moe_weights& wv, const PrefillViews& v, uint32_t rows, hipStream_t st) {
    const uint32_t assignments = rows * wv.top_k, bound = plan_item_bound(wv.experts, assignments, kPfTile);
    launch_plan(v.routes, wv.experts, assignments, kPfTile, bound, v.plan, st);
    PrefillArgs a{};
    a.top_k = wv.top_k; a.exp_kind = wv.exp_kind; a.swiglu_limit = wv.swiglu_limit; a.x = static_cast<const uint8_t*>(v.input); a.x_stride = v.input_stride;
    uint8_t* ws = static_cast<uint8_t*>(v.h_f16);
    a.h = reinterpret_cast<_Float16*>(ws); a.h_lo = reinterpret_cast<_Float16*>(ws + pf_h_plane_bytes(assignments, wv.ffn));
    a.h_sums = ws + pf_h_bytes(assignments, wv.ffn);
    uint8_t* x_sums = a.h_sums + static_cast<size_t>(assignments) * pf_sum_row_bytes(wv.ffn);
    a.x_sums = x_sums;
    a.rawdots = v.rawdots; a.rawdots_rs = v.rawdots_rs; a.rawdots_bf16 = v.rawdots_bf16; a.plan = v.plan; a.experts = wv.experts; a.assignments = assignments;
    a.status = v.status; a.status_rs = v.status_rs; a.job_status = v.job_status; a.items = bound;
    token_sums_kernel<<<rows, 256, 0, st>>>(a.x, a.x_stride, wv.hidden, x_sums);
    if (pf_sum_slots(wv.ffn) != wv.ffn / 32U) clear_sum_padding_kernel<<<assignments, 64, 0, st>>>(a.h_sums, wv.ffn);
    const uint32_t items_at = plan_items_at(wv.experts, assignments), order_at = plan_order_at(wv.experts), item_slots = (bound + 7U) / 8U * 8U;
    // persistent workgroups, one per compute unit (the kernels' LDS use allows no second one)
    const uint32_t cus = compute_units();
    const uint32_t resident = (cus > 8U ? cus : 256U) & ~7U;
    const auto grid_of = [&](uint32_t units) { return units < resident ? units : resident; };
    // gate / up + SwiGLU. Q4_K tensors: every wave expands its own rows in registers (prefill_reg.hpp); Q5_K / Q8_0: the loader /
    // multiplier kernel (prefill_f16.hpp). Both leave h as two fp16 planes and its sub-block sums.
    a.wa = wv.gate; a.wb = wv.up; a.expert_stride = wv.gate_expert_stride; a.row_stride = wv.gate_row_stride; a.k = wv.hidden; a.features = wv.ffn;
    a.lo_pass = 0;
    if (wv.gate_type == MI355_TYPE_Q4_K && wv.ffn % 128U == 0) {
        a.tiles = wv.ffn / 128U; a.units = item_slots * a.tiles;
        prefill_reg_kernel<0><<<grid_of(a.units), kRgThreads, 0, st>>>(a, items_at, order_at);
    } else {
        a.tiles = wv.ffn / 64U; a.units = item_slots * a.tiles;
        if (wv.gate_type == MI355_TYPE_Q8_0) prefill_f16_kernel<0, 1><<<grid_of(a.units), kPfThreads, 0, st>>>(a, items_at, order_at);
        else if (wv.gate_type == MI355_TYPE_Q5_K) prefill_f16_kernel<0, 2><<<grid_of(a.units), kPfThreads, 0, st>>>(a, items_at, order_at);
        else prefill_f16_kernel<0, 0><<<grid_of(a.units), kPfThreads, 0, st>>>(a, items_at, order_at);
    }
    // down rows: h enters as hi + lo. The register-operand kernel multiplies both planes in one sweep of the weights; the loader /
    // multiplier kernel runs a second pass over the lo plane that adds to the first pass's outputs.
    a.wa = wv.down; a.wb = nullptr; a.expert_stride = wv.down_expert_stride; a.row_stride = wv.down_row_stride; a.k = wv.ffn; a.features = wv.hidden;
    if (wv.down_type == MI355_TYPE_Q4_K && wv.hidden % 256U == 0) {
        a.tiles = wv.hidden / 256U; a.units = item_slots * a.tiles;
        prefill_reg_kernel<1><<<grid_of(a.units), kRgThreads, 0, st>>>(a, items_at, order_at);
    } else {
        a.tiles = wv.hidden / 128U; a.units = item_slots * a.tiles;
        for (uint32_t pass = 0; pass < 2U; ++pass) {
            a.lo_pass = pass;
            if (wv.down_type == MI355_TYPE_Q8_0) prefill_f16_kernel<1, 1><<<grid_of(a.units), kPfThreads, 0, st>>>(a, items_at, order_at);
            else if (wv.down_type == MI355_TYPE_Q5_K) prefill_f16_kernel<1, 2><<<grid_of(a.units), kPfThreads, 0, st>>>(a, items_at, order_at);
            else prefill_f16_kernel<1, 0><<<grid_of(a.units), kPfThreads, 0, st>>>(a, items_at, order_at);
        }
    }
    STRIX_LAUNCHED("moe prefill f16");
    return MI355_OK;
}
}  // namespace
extern "C" {

int32_t mi355_moe_enqueue_prefill_f16(const mi355_moe_weights* w, const mi355_moe_rows* r, uint32_t rows, uint32_t form, mi355_stream stream) {
    mi355_moe_weights wv;
    if (const int32_t rc = check_moe(w, r, rows, wv, kPrefillClass)) return rc;
    STRIX_REQUIRE(form <= MI355_COMBINE_NONE, "moe prefill: unknown combine form");
    STRIX_REQUIRE(r->input && r->input_kind == MI355_INPUT_F16, "moe prefill: the fp16 form takes fp16 input rows");
    STRIX_REQUIRE(r->input_stride % 16U == 0 && aligned(r->input, 16), "moe prefill: input rows must be 16-byte aligned");
    STRIX_REQUIRE(r->h_f16 && aligned(r->h_f16, 16), "moe prefill: h_f16 workspace is null or misaligned");
    STRIX_REQUIRE(rows <= 65535U, "moe prefill: at most 65535 rows per call");
    STRIX_REQUIRE(wv.hidden % 128U == 0 && wv.ffn % 64U == 0, "moe prefill: hidden must be a multiple of 128, ffn of 64");
    hipStream_t st = hs(stream);
    clear_validate_kernel<<<rows, 64, 0, st>>>(r->routes, r->route_weights, wv.experts, wv.top_k, r->status, r->job_status);
    const PrefillViews v{r->input, r->input_stride, dense_routes(r->routes, wv.top_k), r->status, 4, r->job_status, r->rawdots, 0, 0U, r->plan, r->h_f16};
    if (const int32_t rc = enqueue_prefill_core(wv, v, rows, st)) return rc;
    if (form == MI355_COMBINE_NONE) return MI355_OK;
    return mi355_moe_enqueue_merge(w, r, rows, form, stream);
}

int32_t mi355_swiglu_quantize(const float* gate, const float* up, uint32_t rows, uint32_t ffn, uint32_t exp_kind, float swiglu_limit,
                              int8_t* codes, float* deltas, int32_t* sums, float* h_out, uint32_t* status, mi355_stream stream) {
    STRIX_REQUIRE(ffn % 32U == 0, "swiglu: ffn must be a multiple of 32");
    STRIX_REQUIRE(exp_kind <= MI355_EXP_DECLARED, "swiglu: unknown exp kind");
    if (swiglu_limit == 0.0F) swiglu_limit = INFINITY;
    STRIX_REQUIRE(swiglu_limit > 0.0F, "swiglu: swiglu_limit must be +infinity (none) or finite and positive");
    if (rows == 0 || ffn == 0) return MI355_OK;
    STRIX_REQUIRE(gate && up && codes && deltas && sums, "swiglu: null pointer");
    STRIX_REQUIRE(rows <= 65535U, "swiglu: at most 65535 rows per call");
    swiglu_quantize_kernel<<<dim3((ffn / 32U + 7U) / 8U, rows), 256, 0, hs(stream)>>>(gate, up, ffn, exp_kind, swiglu_limit, codes, deltas, sums, h_out, status, nullptr);
    STRIX_LAUNCHED("swiglu_quantize");
    return MI355_OK;
}

// ------------------------------------------------------------------------------------------------------------------
// mi355_moe_enqueue_layer for callers that cannot allocate: every work buffer of the layer (router scores, the A8 images
// of the input and of h, the expert plan, the unweighted down outputs, the job status word) lives in a file-scope device
// array of a fixed size instead of caller memory. Each device holds its own copy of that array; its address on a device is
// looked up once (hipGetSymbolAddress with that device current) and kept, and only that address - never the array's name -
// is handed to kernels.
namespace {
constexpr uint32_t kStaticRows = 16, kStaticTopK = 8, kStaticHidden = 8192, kStaticFfn = 4096, kStaticExperts = 1024;
constexpr uint32_t kStaticAssignments = kStaticRows * kStaticTopK;
constexpr size_t align256(size_t v) { return (v + 255U) & ~static_cast<size_t>(255U); }
constexpr size_t kStaticPlanAt = 0;
constexpr size_t kStaticJobAt = kStaticPlanAt + align256(4U * static_cast<size_t>(plan_words_total(kStaticExperts, kStaticAssignments)));
constexpr size_t kStaticScoresAt = kStaticJobAt + 256U;
constexpr size_t kStaticCodesAt = kStaticScoresAt + align256(4U * static_cast<size_t>(kStaticRows) * kStaticExperts);
constexpr size_t kStaticDeltasAt = kStaticCodesAt + align256(static_cast<size_t>(kStaticRows) * kStaticHidden);
constexpr size_t kStaticSumsAt = kStaticDeltasAt + align256(4U * static_cast<size_t>(kStaticRows) * (kStaticHidden / 32U));
constexpr size_t kStaticDownCodesAt = kStaticSumsAt + align256(4U * static_cast<size_t>(kStaticRows) * (kStaticHidden / 32U));
constexpr size_t kStaticDownDeltasAt = kStaticDownCodesAt + align256(static_cast<size_t>(kStaticAssignments) * kStaticFfn);
constexpr size_t kStaticDownSumsAt = kStaticDownDeltasAt + align256(4U * static_cast<size_t>(kStaticAssignments) * (kStaticFfn / 32U));
constexpr size_t kStaticRawdotsAt = kStaticDownSumsAt + align256(4U * static_cast<size_t>(kStaticAssignments) * (kStaticFfn / 32U));
constexpr size_t kStaticBytes = kStaticRawdotsAt + align256(4U * static_cast<size_t>(kStaticAssignments) * kStaticHidden);    // about 5.1 MB
}  // namespace
static __device__ __align__(256) unsigned char scratch[kStaticBytes];     // zero at load: the plan's ticket words start at zero
namespace {
std::atomic<unsigned char*> g_scratch_of_device[64];
// the array's address on the current device (looked up on the first call there); nullptr with the reason in g_error
unsigned char* scratch_on_current_device() {
    int device = -1;
    const hipError_t e0 = hipGetDevice(&device);
    if (e0 != hipSuccess) { hip_fail(e0, "static workspace: hipGetDevice"); return nullptr; }
    if (device < 0 || device >= 64) { fail(MI355_E_UNSUPPORTED, "static workspace: device ordinal beyond 63"); return nullptr; }
    unsigned char* known = g_scratch_of_device[device].load(std::memory_order_acquire);
    if (known) return known;
    void* found = nullptr;
    const hipError_t e1 = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
    if (e1 != hipSuccess || !found) { hip_fail(e1, "static workspace: hipGetSymbolAddress"); return nullptr; }
    g_scratch_of_device[device].store(static_cast<unsigned char*>(found), std::memory_order_release);   // (a racing first call stores the same address)
    return static_cast<unsigned char*>(found);
}
__global__ __launch_bounds__(256) void zero_words_kernel(uint32_t* words, uint32_t count) {
    const uint32_t i = blockIdx.x * 256U + threadIdx.x;
    if (i < count) words[i] = 0U;
}
// The plan words every launch expects to find zero and leaves zero (tickets, arrival counts, tags, the epoch): all zero is the
// state of a freshly loaded library. A kernel store, so that the call may sit inside a captured graph.
int32_t static_plan_reset(unsigned char* ws, hipStream_t st) {
    zero_words_kernel<<<(kPlanOffsetsAt - kPlanTicketsAt + 255U) / 256U, 256, 0, st>>>(reinterpret_cast<uint32_t*>(ws + kStaticPlanAt) + kPlanTicketsAt,
                                                                                  kPlanOffsetsAt - kPlanTicketsAt);
    STRIX_LAUNCHED("static workspace reset");
    return MI355_OK;
}
}  // namespace

int32_t mi355_static_workspace_prepare(mi355_stream stream) {
    unsigned char* ws = scratch_on_current_device();
    if (!ws) return g_error.rfind("static workspace: device", 0) == 0 ? MI355_E_UNSUPPORTED : MI355_E_HIP;
    return static_plan_reset(ws, hs(stream));
}

int32_t mi355_moe_enqueue_layer_static(const mi355_route_policy* p, const float* router_weight, const float* logit_bias,
                                       const mi355_moe_weights* w, const void* input, uint32_t input_kind, uint64_t input_stride,
                                       uint32_t rows, uint32_t* routes, float* route_weights, uint32_t* status, const float* base,
                                       float* output, uint64_t output_stride, uint32_t form, mi355_stream stream) {
    STRIX_REQUIRE(p && w, "moe layer (static workspace): null policy or weights");
    STRIX_REQUIRE(rows >= 1U && rows <= kStaticRows, "moe layer (static workspace): rows must be within 1..16");
    STRIX_REQUIRE(w->top_k >= 1U && w->top_k <= kStaticTopK, "moe layer (static workspace): top_k must be within 1..8");
    STRIX_REQUIRE(w->hidden <= kStaticHidden && w->ffn <= kStaticFfn && w->experts <= kStaticExperts,
                  "moe layer (static workspace): hidden <= 8192, ffn <= 4096 and experts <= 1024 are the limits of the built-in workspace");
    STRIX_REQUIRE(routes && route_weights && status && output && input, "moe layer (static workspace): null row view");
    unsigned char* ws = scratch_on_current_device();
    if (!ws) return g_error.rfind("static workspace: device", 0) == 0 ? MI355_E_UNSUPPORTED : MI355_E_HIP;
    mi355_moe_rows r{};
    r.input = input; r.input_kind = input_kind; r.input_stride = input_stride;
    r.routes = routes; r.route_weights = route_weights; r.status = status; r.base = base; r.output = output; r.output_stride = output_stride;
    r.plan = reinterpret_cast<uint32_t*>(ws + kStaticPlanAt);
    r.job_status = reinterpret_cast<uint32_t*>(ws + kStaticJobAt);
    r.codes = reinterpret_cast<int8_t*>(ws + kStaticCodesAt);
    r.deltas = reinterpret_cast<float*>(ws + kStaticDeltasAt);
    r.sums = reinterpret_cast<int32_t*>(ws + kStaticSumsAt);
    r.down_codes = reinterpret_cast<int8_t*>(ws + kStaticDownCodesAt);
    r.down_deltas = reinterpret_cast<float*>(ws + kStaticDownDeltasAt);
    r.down_sums = reinterpret_cast<int32_t*>(ws + kStaticDownSumsAt);
    r.rawdots = reinterpret_cast<float*>(ws + kStaticRawdotsAt);
    const int32_t rc = mi355_moe_enqueue_layer(p, router_weight, logit_bias, reinterpret_cast<float*>(ws + kStaticScoresAt), w, &r, rows, form, stream);
    // a launch that failed part-way (MI355_E_HIP) may have left counters of the shared plan half-way: put them back to zero for the
    // next call (an admission failure enqueued nothing)
    if (rc == MI355_E_HIP) {
        const std::string first = g_error;
        (void)static_plan_reset(ws, hs(stream));
        g_error = first;
    }
    return rc;
}

}  // extern "C"

#include "a8_contract.hpp"
#include "rows_forms.hpp"
#include "combine_forms.hpp"
#include "shared_gate.hpp"
#include "gguf_reader.hpp"
