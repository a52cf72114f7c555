// Early routes for decode batches: the expert choice leaves the critical path of the layer.
//
// The reference's logits are one ascending fma chain per (row, expert) - `hidden` dependent operations, microseconds of
// latency during which nothing else of the layer can start. The expert *ids* do not need those bits: a dot product in any
// summation order picks the same top-k except where two logits lie within rounding of each other. So the layer runs as
//   1. front launch (layer_front_kernel): early blocks compute the logits as lane-parallel sums (one wave per row and four
//      experts, operands straight into registers) and pick the top-k, the A8 prologue rides beside them, projection blocks
//      sweep gate / up on the early ids as soon as those are tagged, and side blocks run the exact router (the chain, the
//      softmax, the selection, the weights - the reference's bits, written to the caller's ids / weights / scores); the side
//      block that finishes a row compares its exact ids with the early ones and, where they differ, waits for that
//      assignment's speculative waves and repairs the assignment (a copy of the h image the row already holds under another
//      slot, or a sweep on the exact expert) and writes the work items with the exact experts;
//   2. down rows + combine on work items that are exact by then.
// Every output is the exact router's; the early choice only decides which weights stream first.
// Reference (the bits kept): tests/hip_moe_route_launcher_tests.hip:281-330, include/strix/moe/route_policy.hpp:99-156.
#pragma once
#include "route_wave.hpp"
#include "q4k_rows.hpp"

namespace strix950 {

constexpr uint32_t kEarlyExperts = 4;         // experts per early block
constexpr uint32_t kEarlySpinLimit = 1U << 20;      // polls of the selecting block (cannot run out, short of a lost launch)

// ---------------------------------------------------------------------------------------------------- early logits
// Lane l owns features 8 l .. 8 l + 7 of every run of 512; four runs are requested together (36 loads in flight).
template <int KIND>
__device__ __forceinline__ void early_logits_block(const RouteArgs& a, uint32_t row, uint32_t e0, uint32_t epoch) {
    const uint32_t lane = threadIdx.x & 63U;
    float acc[kEarlyExperts];
    const float* wrow[kEarlyExperts];
#pragma unroll
    for (uint32_t i = 0; i < kEarlyExperts; ++i) {
        acc[i] = 0.0F;
        const uint32_t e = e0 + i < a.p.experts ? e0 + i : a.p.experts - 1U;
        wrow[i] = a.wr + static_cast<size_t>(e) * a.hidden;
    }
    const uint8_t* xrow = a.x + row * a.x_stride;
    for (uint32_t k0 = 0; k0 < a.hidden; k0 += 2048U) {
        f32x4 wv[4][kEarlyExperts][2];
        u32x4 xr[4][2];
        bool ok[4];
#pragma unroll
        for (uint32_t s = 0; s < 4U; ++s) {
            const uint32_t k = k0 + 512U * s + 8U * lane;
            ok[s] = k < a.hidden;
            const uint32_t kk = ok[s] ? k : 0U;
#pragma unroll
            for (uint32_t i = 0; i < kEarlyExperts; ++i) {
                wv[s][i][0] = *reinterpret_cast<const f32x4*>(wrow[i] + kk);
                wv[s][i][1] = *reinterpret_cast<const f32x4*>(wrow[i] + kk + 4U);
            }
            if constexpr (KIND == 0) {
                xr[s][0] = *reinterpret_cast<const u32x4*>(xrow + 4U * kk);
                xr[s][1] = *reinterpret_cast<const u32x4*>(xrow + 4U * kk + 16U);
            } else {
                xr[s][0] = *reinterpret_cast<const u32x4*>(xrow + 2U * kk);
            }
        }
#pragma unroll
        for (uint32_t s = 0; s < 4U; ++s) {
            float f[8];
            if constexpr (KIND == 0) {
#pragma unroll
                for (int q = 0; q < 4; ++q) { f[q] = f_of(xr[s][0][q]); f[4 + q] = f_of(xr[s][1][q]); }
            } else {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint32_t h = xr[s][0][q];
                    if constexpr (KIND == 1) { f[2 * q] = half_bits_to_float(h & 0xffffU); f[2 * q + 1] = half_bits_to_float(h >> 16); }
                    else { f[2 * q] = f_of(h << 16); f[2 * q + 1] = f_of(h & 0xffff0000U); }
                }
            }
            if (!ok[s]) {
#pragma unroll
                for (int q = 0; q < 8; ++q) f[q] = 0.0F;
            }
#pragma unroll
            for (uint32_t i = 0; i < kEarlyExperts; ++i) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    acc[i] = __builtin_fmaf(f[q], wv[s][i][0][q], acc[i]);
                    acc[i] = __builtin_fmaf(f[4 + q], wv[s][i][1][q], acc[i]);
                }
            }
        }
    }
    // a logit travels as one 64-bit word {this call's epoch, its bits}: the row's selecting block reads the words until all carry the
    // epoch - no count, no wait for an acknowledgement in between
    unsigned long long* out = reinterpret_cast<unsigned long long*>(a.early_logits) + static_cast<size_t>(row) * (a.early_stride / 2U);
#pragma unroll
    for (uint32_t i = 0; i < kEarlyExperts; ++i) {
        float v = acc[i];
        v = v + xor1_f(v); v = v + xor2_f(v); v = v + xor4_f(v); v = v + xor8_f(v); v = v + xor16_f(v);
        v = v + __shfl_xor(v, 32);
        const uint32_t e = e0 + i;
        if (lane == i && e < a.p.experts) {
            if (a.bias) v = v + a.bias[e];
            // test knob: displaces the early logits (never the exact ones), so that early and exact ids differ
            if (a.early_perturb) v = v + static_cast<float>(a.early_perturb) * 1e-3F * (static_cast<float>((e * 2654435761U) >> 28) - 8.0F);
            __hip_atomic_store(out + e, (static_cast<unsigned long long>(epoch) << 32) | b_of(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// ---------------------------------------------------------------------------------------------------- hand-off between workgroups
// The launches of this file exchange a few words between workgroups: logits, a per-row arrival count, per-assignment counts.
// All of them are read and written by device-scope atomic operations only (they are performed at the memory side, past the
// per-XCD caches), so no cache write-back or invalidation is needed around them: a producer waits until its stores have been
// acknowledged and then counts itself in; the consumer's reads follow its own count operation in program order. Each row's
// count sits in a 128-byte line of its own (32 workgroups counting into one line cost about 0.3 us; all rows' counts in one
// line were measured at 3 us).
__device__ __forceinline__ void stores_acknowledged() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// true in every lane of the one-wave workgroup that arrives last of `parties`; that workgroup leaves the count zero again
__device__ __forceinline__ bool arrive_last(uint32_t* count, uint32_t parties) {
    stores_acknowledged();
    uint32_t seen = 0;
    if ((threadIdx.x & 63U) == 0) seen = __hip_atomic_fetch_add(count, 1U, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    seen = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(seen)));
    asm volatile("" ::: "memory");
    if (seen != parties - 1U) return false;
    if ((threadIdx.x & 63U) == 0) __hip_atomic_store(count, 0U, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return true;
}

// top-k of one row's early logits: greater logit first, lower id on ties. Returns, in lane k < top_k, the expert of slot k.
// A pass = one wave-wide maximum of 32-bit keys (the logit's bits made order preserving) by DPP row shifts and broadcasts, then
// the lowest id among the lanes that hold it.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t max_step_u32(uint32_t v) {
    const uint32_t o = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, ROW_MASK, 0xF, false));
    return o > v ? o : v;
}
__device__ __forceinline__ uint32_t max_wave_u32(uint32_t v) {
    v = max_step_u32<0x111, 0xF>(v); v = max_step_u32<0x112, 0xF>(v); v = max_step_u32<0x114, 0xF>(v); v = max_step_u32<0x118, 0xF>(v);
    v = max_step_u32<0x142, 0xA>(v); v = max_step_u32<0x143, 0xC>(v);
    return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), 63));
}
// ok (all lanes): every logit of the row arrived within the bounded wait.
template <uint32_t PER>
__device__ __forceinline__ uint32_t early_select_row_per(const RouteArgs& a, uint32_t row, uint32_t epoch, bool& ok) {
    const uint32_t lane = threadIdx.x & 63U, E = a.p.experts, K = a.p.top_k;
    const unsigned long long* z = reinterpret_cast<const unsigned long long*>(a.early_logits) + static_cast<size_t>(row) * (a.early_stride / 2U);
    uint32_t key[PER];
    uint64_t missing = ~0ULL;
    for (uint32_t spins = 0; spins < kEarlySpinLimit && missing; ++spins) {
        bool mine = false;
#pragma unroll
        for (uint32_t i = 0; i < PER; ++i) {
            const uint32_t e = lane + 64U * i;
            key[i] = 0;                                                          // 0 = absent or taken
            if (e < E) {
                const unsigned long long word = __hip_atomic_load(z + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);       // written by other workgroups of this launch
                mine = mine || static_cast<uint32_t>(word >> 32) != epoch;
                const uint32_t b = static_cast<uint32_t>(word);
                const uint32_t sortable = (b & 0x80000000U) ? ~b : (b | 0x80000000U);
                key[i] = sortable ? sortable : 1U;
            }
        }
        missing = __ballot(mine);
        if (missing) __builtin_amdgcn_s_sleep(4);
    }
    ok = missing == 0;
    uint32_t my_id = 0;
#pragma unroll 1
    for (uint32_t k = 0; k < K; ++k) {
        uint32_t best = key[0];
#pragma unroll
        for (uint32_t i = 1; i < PER; ++i) best = key[i] > best ? key[i] : best;
        best = max_wave_u32(best);
        uint32_t id = 0;
        bool found = false;
#pragma unroll
        for (uint32_t i = 0; i < PER; ++i) {
            const uint64_t holders = __ballot(key[i] == best);
            if (!found && holders) {
                found = true;
                const uint32_t owner = static_cast<uint32_t>(__ffsll(static_cast<long long>(holders))) - 1U;
                id = owner + 64U * i;
                if (lane == owner) key[i] = 0;
            }
        }
        if (lane == k) my_id = id;
    }
    return my_id;
}
__device__ __forceinline__ uint32_t early_select_row(const RouteArgs& a, uint32_t row, uint32_t epoch, bool& ok) {
    const uint32_t E = a.p.experts;
    if (E <= 128U) return early_select_row_per<2>(a, row, epoch, ok);
    if (E <= 256U) return early_select_row_per<4>(a, row, epoch, ok);
    if (E <= 512U) return early_select_row_per<8>(a, row, epoch, ok);
    return early_select_row_per<16>(a, row, epoch, ok);
}

// ---------------------------------------------------------------------------------------------------- the exact chain as a side block
// The reference's chain inside the layer launch: a one-wave block that owns two experts of one row. Its two router-weight rows
// are requested whole at the block's start (one 10,240-byte LDS object each, the launch's two ring slots), so once they have
// landed the chain no longer touches memory - the other waves of the launch saturate it. Lane 0 / 1 run the chains of the two
// experts, the weight operand by 128-bit LDS reads 16 features ahead.
//   fp16 / bf16 rows: the row rides along as 16-bit values in the 2 KB behind each weight row (features 0..1023 behind the
//     first, the rest behind the second); per 16 features one 16-bit LDS read leaves feature k + t in lane t of every row of 16
//     lanes, widened once, and the fma takes it by a DPP row broadcast (chain_run of route_wave.hpp).
//   fp32 rows do not fit beside the weights: they sit in registers (lane L holds features 32 L .. 32 L + 31) and reach the fma
//     as a scalar operand through v_readlane (about four times the latency per step; still off the layer's critical path).
// Needs hidden <= 2048, hidden % 64 == 0.
constexpr uint32_t kSideExperts = 2, kSideMaxHidden = 2048, kSideSlotBytes = 10240, kSideRowBytes = 8192;

__device__ __forceinline__ void side_copy16(const void* src, uint32_t lds_at) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_at), "v"(src) : "memory", "m0");
}

template <int KIND>
__device__ __forceinline__ void side_chain_block(lds_u8* ring0, lds_u8* ring1, const RouteArgs& a, uint32_t row, uint32_t e0) {
    const uint32_t lane = threadIdx.x & 63U, row_bytes = a.hidden * 4U;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    lds_u8* const ring[kSideExperts] = {ring0, ring1};
#pragma unroll
    for (uint32_t i = 0; i < kSideExperts; ++i) {
        const uint32_t e = e0 + i < a.p.experts ? e0 + i : a.p.experts - 1U;
        const uint8_t* src = reinterpret_cast<const uint8_t*>(a.wr + static_cast<size_t>(e) * a.hidden) + 16U * lane;
        const uint32_t at = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(ring[i]));
        for (uint32_t off = 0; off < row_bytes; off += 1024U)
            if (off + 16U * lane < row_bytes) side_copy16(src + off, at + off);
    }
    const uint8_t* xrow = a.x + row * a.x_stride;
    float acc = 0.0F;
    const float* wrow = reinterpret_cast<const float*>((lane & 1U) ? (uint8_t*)ring1 : (uint8_t*)ring0);
    if constexpr (KIND == 0) {
        float xf[32];
        const bool mine = 32U * lane < a.hidden;
        const uint32_t k = mine ? 32U * lane : 0U;
        f32x4 v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = *reinterpret_cast<const f32x4*>(xrow + 4U * k + 16U * i);
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) xf[4 * i + q] = mine ? v[i][q] : 0.0F;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        const uint32_t blocks = a.hidden / 32U;
        f32x4 wv[8], wn[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) wv[i] = *reinterpret_cast<const f32x4*>(wrow + 4 * i);
        for (uint32_t L = 0; L < blocks; ++L) {
            const uint32_t Ln = L + 1U < blocks ? L + 1U : L;
#pragma unroll
            for (int i = 0; i < 8; ++i) wn[i] = *reinterpret_cast<const f32x4*>(wrow + 32U * Ln + 4 * i);
#pragma unroll
            for (int j = 0; j < 32; ++j) {
                const float xs = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, xf[j]), static_cast<int>(L)));
                acc = __builtin_fmaf(xs, wv[j / 4][j % 4], acc);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) wv[i] = wn[i];
        }
    } else {
        // the row as it is (2 bytes per feature) behind the weight rows: 1024 features = 2 KB = two copies of 64 x 16 bytes each
#pragma unroll
        for (uint32_t i = 0; i < kSideExperts; ++i) {
            const uint32_t at = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(ring[i])) + kSideRowBytes;
#pragma unroll
            for (uint32_t j = 0; j < 2U; ++j) {
                const uint32_t k = 1024U * i + 512U * j + 8U * lane;
                if (k < a.hidden) side_copy16(xrow + 2U * k, at + 1024U * j);
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        const uint32_t t = lane & 15U;
        // the 16-bit value of feature k + t as read; it is widened only when its 16 steps are about to run, so the read's latency
        // hides behind the steps in front of it
        auto raw_of = [&](uint32_t k) {
            return static_cast<uint32_t>(*reinterpret_cast<const uint16_t*>((k < 1024U ? (uint8_t*)ring0 : (uint8_t*)ring1) + kSideRowBytes + 2U * ((k & 1023U) + t)));
        };
        auto widen = [&](uint32_t h) {
            if constexpr (KIND == 1) return half_bits_to_float(h);
            else return f_of(h << 16);
        };
        // Operands are fetched 48 features ahead of the chain (four buffers): with one step of 16 ahead every step waited for its
        // LDS reads (128 waits of ~200 cycles: the loop took 12.6 us inside the layer launch against ~5 us for the 2048 fmas).
        ChainStep S0, S1, S2, S3;
        uint32_t r0, r1, r2, r3;
        auto load = [&](ChainStep& s, uint32_t& raw, uint32_t k) {
            const uint32_t kk = k < a.hidden ? k : a.hidden - 16U;      // (past the end: a valid place, never used)
#pragma unroll
            for (uint32_t i = 0; i < 4U; ++i) s.w[i] = *reinterpret_cast<const f32x4*>(wrow + kk + 4U * i);
            raw = raw_of(kk);
        };
        load(S0, r0, 0U); load(S1, r1, 16U); load(S2, r2, 32U);
        for (uint32_t k = 0; k < a.hidden; k += 64U) {      // hidden % 64 == 0 on this path
            load(S3, r3, k + 48U);
            __builtin_amdgcn_sched_barrier(0);
            S0.x = widen(r0);
            acc = chain_run(S0, acc);
            __builtin_amdgcn_sched_barrier(0);
            load(S0, r0, k + 64U);
            __builtin_amdgcn_sched_barrier(0);
            S1.x = widen(r1);
            acc = chain_run(S1, acc);
            __builtin_amdgcn_sched_barrier(0);
            load(S1, r1, k + 80U);
            __builtin_amdgcn_sched_barrier(0);
            S2.x = widen(r2);
            acc = chain_run(S2, acc);
            __builtin_amdgcn_sched_barrier(0);
            load(S2, r2, k + 96U);
            __builtin_amdgcn_sched_barrier(0);
            S3.x = widen(r3);
            acc = chain_run(S3, acc);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    const uint32_t e = e0 + lane;
    if (lane < kSideExperts && e < a.p.experts)
        __hip_atomic_store(a.scores + static_cast<size_t>(row) * a.p.experts + e, a.bias ? acc + a.bias[e] : acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace strix950
