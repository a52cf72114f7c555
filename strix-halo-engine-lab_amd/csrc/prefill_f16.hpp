// Prefill form of the routed experts for gfx950: an expert-grouped GEMM on the matrix cores. This is the path's second
// arithmetic class (the reference's FAST forms, include/strix/cuda/qwen_moe.hpp:100-101 "bit-changing"); its parity target
// is the exact-weight product (include/strix/ds41_layer.hpp:96-121) within the stated tolerance, not the integer-dot
// class's bits.
//
// Arithmetic. A Q4_K weight is w = d_b (sc_j q) - dmin_b m_j (super-block b of 256, sub-block j of 32, q a nibble;
// src/ggml_dequant.cpp:119-130). The kernel never rounds a weight to fp16. For output feature f and token t
//   out[t][f] = sum_b d_b[f] * P_b[t][f]  +  sum_(b,j) S_bj[t] * M_bj[f],
//   P_b = sum_(k in b) (sc_j q_k) x_k[t],   S_bj[t] = sum_(k in sub-block j of b) x_k[t],   M_bj[f] = -(dmin_b m_j).
// sc_j q_k is an integer <= 945: exact in fp16, so P_b is an fp16 MFMA with fp32 accumulation whose only rounding is the
// fp32 accumulation; d_b is applied in fp32 once per super-block. The second sum is a product over K / 32 sub-blocks:
// S and M are each carried as two fp16 numbers (hi = fp16(v), lo = fp16(v - hi)) and multiplied by three MFMAs per 16
// sub-blocks (hi*hi + lo*hi + hi*lo). S of the input rows comes from token_sums_kernel, S of h from the epilogue of
// the gate / up launch.
//
// Work decomposition. The expert plan cuts every expert's assignments into items of at most 128 rows. A 512-thread
// workgroup owns (item, 64 output features of gate AND up) or (item, 128 output features of down): 128 weight rows x
// 128 tokens, K walked in steps of 64 (one pair of Q4_K sub-blocks: 32 quant bytes whose low / high nibbles are
// sub-blocks 2p / 2p + 1). Waves 0-3 are loaders, waves 4-7 multipliers (one of each per SIMD):
//   * token rows go from global memory straight into a 4-stage LDS ring (global_load_lds by the multiplier waves, 3 steps ahead of their use);
//   * a loader thread owns (weight row, 16 quant bytes): a super-block's raw bytes are fetched into registers five steps
//     ahead, turned into
//     32 fp16 integers sc q with v_perm / v_and_or / v_pk_fma_f16 (1024 + q is the fp16 bit pattern 0x6400 | q, and
//     fma(1024 + q, sc, -1024 sc) = sc q exactly) and stored in a double-buffered LDS tile; d_b, and every two
//     super-blocks the M tile, go to small LDS arrays; the S tile of the same 16 sub-blocks is copied by global_load_lds;
//   * a multiplier wave holds a 64 x 64 quarter (2 x 2 MFMA tiles, A = tokens, B = weights: a lane of the result is
//     one feature, so d_b is one register per tile row) in two sets of accumulators: P (cleared every super-block) and
//     the running sum.
// LDS tiles are [row][64 halves] with a 128-byte pitch and the 16-byte pieces of a row XOR-swizzled by (row / 2) % 8: a
// 128-bit LDS access is served sixteen lanes at a time over 64 banks, and sixteen consecutive rows then cover all banks for
// the MFMA operand reads and the loaders' stores (measured: swizzling by row % 8 instead doubles the conflict cycles), while
// a copy instruction still writes 1 KB of consecutive LDS. One barrier per step.
//
// Workgroups are numbered so that the feature tiles of one item run on one XCD (consecutive workgroup ids go round
// the 8 XCDs): its token rows are then read from HBM once per XCD and served from that XCD's L2 afterwards.
#pragma once
#include "device_math.hpp"
#include "q4k_rows.hpp"
#include <type_traits>

namespace strix950 {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) uint8_t pf_lds;

constexpr uint32_t kPfTile = 128;                 // weight rows and tokens per workgroup tile
constexpr uint32_t kPfStep = 64;                  // K per step
constexpr uint32_t kPfTileBytes = kPfTile * 128U; // one step of a tile: 128 rows x 64 halves
constexpr uint32_t kPfRing = 4;                   // token stages (separate LDS objects: stage = step % 4)
constexpr uint32_t kPfTokenTiles = 2;                // 32-token tiles per multiplier wave: 8 / kPfTokenTiles multiplier waves
constexpr uint32_t kPfThreads = 256U + 64U * (8U / kPfTokenTiles);
constexpr uint32_t kPfTokenAhead = 3;             // steps between a token copy and its use

// sub-block sums of a row: two fp16 planes (hi, lo) of `pf_sum_slots(k)` halves each, the slots past k / 32 zero
__host__ __device__ constexpr uint32_t pf_sum_slots(uint32_t k) { return (k / 32U + 15U) & ~15U; }
__host__ __device__ constexpr size_t pf_sum_row_bytes(uint32_t k) { return 4U * static_cast<size_t>(pf_sum_slots(k)); }
// bytes of the fp16 workspace: h [assignments][ffn], sums of h [assignments], sums of the input rows [rows]
// (two fp16 planes: h = hi + lo)
// (one plane holds a tile of 128 rows more than the assignments: the down kernel reads whole tiles of rows)
__host__ __device__ constexpr size_t pf_h_plane_bytes(uint32_t assignments, uint32_t ffn) { return 2U * (static_cast<size_t>(assignments) + 128U) * ffn; }
__host__ __device__ constexpr size_t pf_h_bytes(uint32_t assignments, uint32_t ffn) { return 2U * pf_h_plane_bytes(assignments, ffn); }
__host__ __device__ constexpr size_t pf_workspace_bytes(uint32_t hidden, uint32_t ffn, uint32_t rows, uint32_t top_k) {
    return pf_h_bytes(rows * top_k, ffn) + static_cast<size_t>(rows) * top_k * pf_sum_row_bytes(ffn) + static_cast<size_t>(rows) * pf_sum_row_bytes(hidden);
}

struct PrefillArgs {
    const uint8_t* wa; const uint8_t* wb;         // MODE 0: gate, up; MODE 1: down (wb unused)
    uint64_t expert_stride, row_stride;           // bytes
    uint32_t k;                                   // K = hidden (MODE 0) or ffn (MODE 1), multiple of 256
    uint32_t features;                            // ffn (MODE 0) or hidden (MODE 1)
    uint32_t top_k, exp_kind;
    float swiglu_limit;                           // the clamp trait of the SwiGLU epilogue (+infinity: none)
    const uint8_t* x; uint64_t x_stride;          // MODE 0: fp16 token rows (bytes); MODE 1: unused
    _Float16* h;                                  // [assignments in plan order][ffn] fp16: written by MODE 0, read by MODE 1
    _Float16* h_lo;                               // the same shape: fp16(h - fp16(h)), so that hi + lo carries h to 22 bits
    uint32_t lo_pass;                             // MODE 1 of prefill_f16_kernel: multiply the lo plane and ADD to the outputs (second pass)
    uint8_t* h_sums;                              // [assignments in plan order] sub-block sums of h: written by MODE 0, read by MODE 1
    const uint8_t* x_sums;                        // [rows] sub-block sums of the input rows (MODE 0)
    float* rawdots;                               // MODE 1: [assignment][hidden]
    const uint32_t* plan; uint32_t experts, assignments;
    uint32_t* status; uint32_t* job_status;
    uint32_t tiles, items, units;                 // feature tiles per item, item bound of the launch, tiles * items rounded up to 8 items
    uint64_t status_rs, rawdots_rs;               // bytes between the rows of status / rawdots; rawdots_rs == 0: dense [assignment][features]
    uint32_t rawdots_bf16;                        // MODE 1: every unweighted output is stored once rounded to bfloat16 (as an fp32 value)
};

// the status word of an assignment's row, and the first of its `features` unweighted outputs
__device__ __forceinline__ uint32_t* pf_status_of(const PrefillArgs& a, uint32_t assignment) {
    return reinterpret_cast<uint32_t*>(reinterpret_cast<uint8_t*>(a.status) + static_cast<size_t>(assignment / a.top_k) * a.status_rs);
}
__device__ __forceinline__ float* pf_rawdots_of(const PrefillArgs& a, uint32_t assignment) {
    if (a.rawdots_rs == 0) return a.rawdots + static_cast<size_t>(assignment) * a.features;
    const uint32_t row = assignment / a.top_k, slot = assignment - row * a.top_k;
    return reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(a.rawdots) + static_cast<size_t>(row) * a.rawdots_rs) + static_cast<size_t>(slot) * a.features;
}
// include/strix/moe/combine.hpp:24-33 (the stored output of a bfloat16 Linear: nearest even, a NaN as it is)
__device__ __forceinline__ float pf_round_bf16(float x) {
    const uint32_t bits = __builtin_bit_cast(uint32_t, x);
    if ((bits & 0x7f800000U) == 0x7f800000U && (bits & 0x7fffffU)) return x;
    return __builtin_bit_cast(float, (bits + 0x7fffU + ((bits >> 16U) & 1U)) & 0xffff0000U);
}

__device__ __forceinline__ uint32_t pack_half2(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(float2v{a, b}, half2v));      // v_cvt_pk_f16_f32: round to nearest even
}
// v -> fp16 hi = fp16(v), lo = fp16(v - hi)
__device__ __forceinline__ void split_half(float v, _Float16& hi, _Float16& lo) {
    hi = static_cast<_Float16>(v);
    lo = static_cast<_Float16>(v - static_cast<float>(hi));
}

// Sub-block sums of fp16 rows: one thread per (row, sub-block of 32), fp32 sum in index order.
__global__ __launch_bounds__(256) void token_sums_kernel(const uint8_t* x, uint64_t x_stride, uint32_t k, uint8_t* sums) {
    const uint32_t row = blockIdx.x, slots = pf_sum_slots(k);
    _Float16* hi = reinterpret_cast<_Float16*>(sums + static_cast<size_t>(row) * pf_sum_row_bytes(k));
    _Float16* lo = hi + slots;
    for (uint32_t s = threadIdx.x; s < slots; s += 256U) {
        float sum = 0.0F;
        if (s < k / 32U) {
            const half8* p = reinterpret_cast<const half8*>(x + static_cast<size_t>(row) * x_stride + 64U * s);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const half8 v = p[i];
#pragma unroll
                for (int j = 0; j < 8; ++j) sum += static_cast<float>(v[j]);
            }
        }
        split_half(sum, hi[s], lo[s]);
    }
}

// Padding slots of the sums of h (ffn / 32 not a multiple of 16) must read as zero.
__global__ __launch_bounds__(64) void clear_sum_padding_kernel(uint8_t* sums, uint32_t k) {
    const uint32_t slots = pf_sum_slots(k), used = k / 32U;
    _Float16* hi = reinterpret_cast<_Float16*>(sums + static_cast<size_t>(blockIdx.x) * pf_sum_row_bytes(k));
    for (uint32_t s = used + threadIdx.x; s < slots; s += 64U) { hi[s] = static_cast<_Float16>(0.0F); hi[slots + s] = static_cast<_Float16>(0.0F); }
}

// Workgroup barrier that orders LDS traffic only. __syncthreads() also waits for every outstanding global memory operation
// of the wave, which would drain the copies and fetches that are in flight for later steps at every barrier; their
// arrival is awaited explicitly where it is needed.
// (A fence on the LDS address space counts the copies' LDS writes and waits for them too, hence the plain instructions:
// LDS stores of this wave complete, barrier; the compiler moves no memory access across the statement.)
__device__ __forceinline__ void pf_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// One global -> LDS copy of 16 bytes per lane (lane l lands at lds_base + 16 l), issued as plain instructions: the
// compiler is not told about it, so it adds no waits of its own around later LDS reads; the arrival of a copy is awaited
// by a counted s_waitcnt before the barrier that publishes the stage.
__device__ __forceinline__ void copy16_to_lds(const uint8_t* src, pf_lds* lds_base) {
    const uint32_t at = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds_base)));
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(at), "v"(src) : "memory", "m0");
}

// byte offset of 16-byte piece `piece` (0..7) of tile row `row`
__device__ __forceinline__ uint32_t pf_at(uint32_t row, uint32_t piece) { return row * 128U + ((piece ^ ((row >> 1) & 7U)) << 4); }

// the loader's per-step global operands
struct PfRaw { u32x4 hd, qs[4], fifth; };    // one super-block of a weight row: header, the thread's 16 quant bytes of its four steps, Q5_K: their fifth bits
struct PfRaw8 { u32x4 a, b; uint32_t c; };   // one Q8_0 block of a weight row as nine aligned words

// FMT 0: Q4_K weights; FMT 2: Q5_K weights (the same block with 32 fifth-bit bytes after the factors, bit j of byte k for
// element k of sub-block j: q = nibble | bit << 4, sc q <= 1953 is still an exact fp16 integer); FMT 1: Q8_0 weights (one
// fp16 d per 32 codes and no minimum, src/ggml_dequant.cpp:84-87: the codes
// are exact fp16 integers, a step is two blocks, and d is applied in fp32 to the product of each block).
template <int MODE, int FMT>
__global__ __launch_bounds__(kPfThreads) void prefill_f16_kernel(PrefillArgs a, uint32_t items_at, uint32_t order_at) {
    __shared__ __attribute__((aligned(16))) uint8_t tok0[kPfTileBytes];                     // token steps: stage s % 4
    __shared__ __attribute__((aligned(16))) uint8_t tok1[kPfTileBytes];
    __shared__ __attribute__((aligned(16))) uint8_t tok2[kPfTileBytes];
    __shared__ __attribute__((aligned(16))) uint8_t tok3[kPfTileBytes];
    __shared__ __attribute__((aligned(16))) uint8_t w_tile[2][kPfTileBytes];                // sc q of one step
    __shared__ __attribute__((aligned(16))) uint8_t s_tile_mem[2][kPfTile * 64U];           // [token][hi 16 | lo 16] sums of 16 sub-blocks
    __shared__ __attribute__((aligned(16))) uint8_t m_tile[2][kPfTile * 64U];               // [feature][hi 16 | lo 16] -(dmin m)
    __shared__ float d_scale[2][2U * kPfTile];                                              // d of one super-block (Q4_K: the first 128) or of a step's two blocks (Q8_0)
    pf_lds* const tok_stage[4] = {(pf_lds*)tok0, (pf_lds*)tok1, (pf_lds*)tok2, (pf_lds*)tok3};
    pf_lds* const s_tile = (pf_lds*)s_tile_mem;

    if (MODE == 1 && (*a.job_status & MI355_STATUS_NONFINITE_PROJECTION)) return;
    const uint32_t* order = a.plan + order_at;
    const bool loader = threadIdx.x < 256U;
    // A workgroup is persistent: it walks the (item, feature tile) units v = blockIdx.x, blockIdx.x + gridDim.x, ... (gridDim.x a
    // multiple of 8). Units v, v + 8, v + 16, ... share an XCD and walk the tiles of one item first, so the workgroups of an
    // XCD work on the same item at the same time. The loaders reach the next unit's prologue (plan and pointer loads, first
    // copies) while the multipliers are still in the epilogue of the current one: nobody reads LDS after a unit's last barrier.
    for (uint32_t unit = blockIdx.x; unit < a.units; unit += gridDim.x) {
    const uint32_t xcd = unit & 7U, q = unit >> 3;
    const uint32_t item_index = (q / a.tiles) * 8U + xcd, tile = q % a.tiles;
    if (item_index >= a.items) continue;
    const uint4 item = *reinterpret_cast<const uint4*>(a.plan + items_at + 4U * item_index);
    const uint32_t e = item.x, begin = item.y, count = item.z - item.y;
    if (count == 0) continue;
    const uint32_t t = loader ? threadIdx.x : threadIdx.x - 256U, lane = t & 63U, wave = t >> 6;      // index within the role
    const uint32_t m0 = tile * (MODE == 0 ? 64U : 128U);
    const uint32_t steps = a.k / kPfStep, blocks = a.k / 256U, steps8 = FMT != 1 ? (steps + 7U) & ~7U : steps;   // K is a multiple of 256: steps of 4
    const size_t sum_row = pf_sum_row_bytes(a.k);

    if (loader) {
        // ---- weight side: row lrow of the tile, quant bytes [16 half, 16 half + 16) of every step
        const uint32_t lrow = 32U * wave + (lane & 31U), half = lane >> 5;
        const uint8_t* wbase = (MODE == 0 && (lrow & 32U)) ? a.wb : a.wa;
        const uint32_t wfeature = MODE == 0 ? 32U * (lrow >> 6) + (lrow & 31U) : lrow;
        const uint8_t* wrow = wbase + static_cast<size_t>(e) * a.expert_stride + static_cast<size_t>(m0 + wfeature) * a.row_stride;
        // ---- token side: copy i of a step moves tile rows 8 (4 i + wave) .. + 8; lane = (row % 8, slot)
        const uint8_t* tsrc[4];
#pragma unroll
        for (uint32_t i = 0; i < 4U; ++i) {
            const uint32_t row = 8U * (4U * i + wave) + (lane >> 3), tok = row < count ? row : count - 1U;
            const uint32_t piece = (lane & 7U) ^ ((row >> 1) & 7U);
            if (MODE == 0) tsrc[i] = a.x + static_cast<size_t>(order[begin + tok] / a.top_k) * a.x_stride + 16U * piece;
            else tsrc[i] = reinterpret_cast<const uint8_t*>((a.lo_pass ? a.h_lo : a.h) + static_cast<size_t>(begin + tok) * a.k) + 16U * piece;
        }
        // ---- sums side: copy c of a group moves pieces 256 c + t; piece = (token, part): part 0, 1 = hi, part 2, 3 = lo
        const uint8_t* ssrc[2];
#pragma unroll
        for (uint32_t c = 0; c < 2U; ++c) {
            const uint32_t piece = 256U * c + t, row = piece >> 2, part = piece & 3U, tok = row < count ? row : count - 1U;
            const uint8_t* base = MODE == 0 ? a.x_sums + static_cast<size_t>(order[begin + tok] / a.top_k) * sum_row
                                            : a.h_sums + static_cast<size_t>(begin + tok) * sum_row;
            ssrc[c] = base + 16U * (part & 1U) + (part >> 1) * (sum_row / 2U);
        }
        const uint32_t last = steps - 1U, last_block = blocks - 1U, last_group = (blocks + 1U) / 2U - 1U;
        // (memory operations are issued unconditionally, indices past the end clamped: see below)
        const auto copy_tokens = [&](uint32_t s, pf_lds* stage) {          // 4 operations: step s -> its stage
            const uint32_t sc = s < last ? s : last;
#pragma unroll
            for (uint32_t i = 0; i < 4U; ++i) copy16_to_lds(tsrc[i] + static_cast<size_t>(sc) * 128U, stage + 1024U * (4U * i + wave));
        };
        if constexpr (FMT == 1) {
            // ---- Q8_0: the thread owns block 2 s + half of every step (34 bytes at a 2-byte boundary). Rows start at 4-byte
            // boundaries, so block `half` starts 2 half bytes past one: nine aligned words cover it. For half 0 they are the
            // words from the block's start (d in the low half of the first, codes from byte 2: every code word straddles two);
            // for half 1 eight words from the first code and the word before them (d in its high half).
            const uint8_t* pa = wrow + 34U * half + 2U * half;
            const uint8_t* pc = half ? pa - 4 : pa + 32;
            const uint32_t straddle = half ? 0U : 2U;
            const auto fetch8 = [&](uint32_t s, PfRaw8& r) {                 // 3 operations
                const uint32_t off = 68U * (s < last ? s : last);
                const uint8_t* qa = pa + off;
                const uint8_t* qc = pc + off;
                asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(r.a) : "v"(qa) : "memory");
                asm volatile("global_load_dwordx4 %0, %1, off offset:16" : "=v"(r.b) : "v"(qa) : "memory");
                asm volatile("global_load_dword %0, %1, off" : "=v"(r.c) : "v"(qc) : "memory");
            };
            uint32_t bias_bits;                                              // per half: 0x6400 | 0x80: 1024 + (code ^ 0x80) = 1152 + code
            asm volatile("v_mov_b32 %0, 0x64806480" : "=v"(bias_bits));
            const _Float16 minus = static_cast<_Float16>(-1152.0F);
            const half2v minus2 = {minus, minus};
            const auto stage8 = [&](uint32_t s, const PfRaw8& r) {
                const uint32_t seq[9] = {r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w, half ? r.b.w : r.c};
                uint32_t out[16];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t codes = __builtin_amdgcn_alignbyte(seq[j + 1], seq[j], straddle);
                    // two signed bytes -> the fp16 integers: 0x6400 | (byte ^ 0x80) is 1152 + code
                    const uint32_t lo = __builtin_amdgcn_perm(0U, codes, 0x0c010c00U) ^ bias_bits;
                    const uint32_t hi = __builtin_amdgcn_perm(0U, codes, 0x0c030c02U) ^ bias_bits;
                    out[2 * j] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2v, lo) + minus2);
                    out[2 * j + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2v, hi) + minus2);
                }
                uint8_t* tile_w = w_tile[s & 1U];
#pragma unroll
                for (uint32_t i = 0; i < 4U; ++i)
                    *reinterpret_cast<u32x4*>(tile_w + pf_at(lrow, 4U * half + i)) = u32x4{out[4 * i], out[4 * i + 1], out[4 * i + 2], out[4 * i + 3]};
                d_scale[s & 1U][kPfTile * half + lrow] = half_bits_to_float(half ? r.c >> 16 : r.a.x & 0xffffU);
            };
            // Schedule of one step: token copy of step + 3 (4 operations), fetch of step + 4 into the slot used up by the
            // previous step's staging (3 operations), stage step + 1 (fetched three steps ago: 21 younger operations),
            // wait for the token copy of step + 1 (issued two steps ago, ahead of that step's fetch: 3 + 14), barrier. The
            // prologue issues the sequence of three steps before the first.
            PfRaw8 raw[4];
            fetch8(0, raw[0]);
            copy_tokens(0, tok_stage[0]); fetch8(1, raw[1]);
            copy_tokens(1, tok_stage[1]); fetch8(2, raw[2]);
            copy_tokens(2, tok_stage[2]); fetch8(3, raw[3]);
            // younger than the first token copy (and than the first fetch before it): 3 + 7 + 7
            asm volatile("s_waitcnt vmcnt(17)" : "+v"(raw[0].a), "+v"(raw[0].b), "+v"(raw[0].c) : : "memory");
            stage8(0, raw[0]);
            pf_barrier();
            for (uint32_t s0 = 0; s0 < steps; s0 += 4U) {
#pragma unroll
                for (uint32_t u = 0; u < 4U; ++u) {
                    const uint32_t s = s0 + u;
                    copy_tokens(s + kPfTokenAhead, tok_stage[(u + kPfTokenAhead) & 3U]);
                    fetch8(s + 4U, raw[u]);
                    PfRaw8& next = raw[(u + 1U) & 3U];
                    asm volatile("s_waitcnt vmcnt(21)" : "+v"(next.a), "+v"(next.b), "+v"(next.c) : : "memory");
                    if (s < last) stage8(s + 1U, next);
                    wait_copies<17>();
                    pf_barrier();
                }
            }
            continue;
        }
        // Every memory operation below is issued unconditionally (indices past the end are clamped: such copies land in
        // stages nobody reads any more), so the number of operations between an issue and the point that needs its data
        // is a compile-time constant and the waits are plain s_waitcnt vmcnt(n) of this code's own: the compiler is not
        // told about these operations, whose bookkeeping across loop iterations it resolves by waiting for all of them.
        const auto copy_sums = [&](uint32_t g) {                           // 2 operations: 16 sub-blocks of group g -> s_tile[g % 2]
            const uint32_t gc = g < last_group ? g : last_group;
#pragma unroll
            for (uint32_t c = 0; c < 2U; ++c)
                copy16_to_lds(ssrc[c] + static_cast<size_t>(gc) * 32U, s_tile + (g & 1U) * (kPfTile * 64U) + 4096U * c + 1024U * wave);
        };
        // 5 operations: a super-block's header and the thread's 16 quant bytes of each of its four steps, issued together
        // (they touch the same two or three cache lines)
        constexpr uint32_t kBlockBytes = FMT == 2 ? 176U : 144U, kQuantsAt = FMT == 2 ? 48U : 16U;
        constexpr uint32_t kFetchOps = FMT == 2 ? 6U : 5U;                 // operations of one fetch (Q5_K: + the fifth bits)
        const auto fetch = [&](uint32_t b, PfRaw& r) {
            const uint8_t* blk = wrow + static_cast<size_t>(b < last_block ? b : last_block) * kBlockBytes;
            const uint8_t* quants = blk + kQuantsAt + 16U * half;
            if (FMT == 2) {
                const uint8_t* bits = blk + 16U + 16U * half;              // fifth bits of elements 16 half .. + 16 of every sub-block
                asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(r.fifth) : "v"(bits) : "memory");
            }
            asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(r.hd) : "v"(blk) : "memory");
            asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(r.qs[0]) : "v"(quants) : "memory");
            asm volatile("global_load_dwordx4 %0, %1, off offset:32" : "=v"(r.qs[1]) : "v"(quants) : "memory");
            asm volatile("global_load_dwordx4 %0, %1, off offset:64" : "=v"(r.qs[2]) : "v"(quants) : "memory");
            asm volatile("global_load_dwordx4 %0, %1, off offset:96" : "=v"(r.qs[3]) : "v"(quants) : "memory");
        };
        // the two constants of the nibble expansion, kept in registers so that mask-and-merge is one v_and_or_b32
        // (as immediates the instruction cannot encode them and the compiler emits two)
        uint32_t nibble_mask, magic_1024;
        if (FMT == 2) asm volatile("s_mov_b32 %0, 0x001f001f" : "=s"(nibble_mask));
        else asm volatile("s_mov_b32 %0, 0x000f000f" : "=s"(nibble_mask));
        asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(magic_1024));
        // (p = step % 4 and the step's parity are compile-time constants at every call)
        const auto stage_weights = [&](uint32_t b, uint32_t p, const u32x4& hd, const u32x4& quants, const u32x4& fifth) {
            const uint32_t sh0 = 16U * (p & 1U), sh1 = sh0 + 8U;
            const uint32_t fa0 = (hd.y >> sh0) & 255U, fc0 = (hd.w >> sh0) & 255U;
            const uint32_t fa1 = (hd.y >> sh1) & 255U, fc1 = (hd.w >> sh1) & 255U;
            const bool low = p < 2U;                          // uniform: p is the same for the whole workgroup
            const uint32_t s0 = low ? (fa0 & 63U) : ((fc0 & 15U) | ((fa0 >> 6) << 4));
            const uint32_t s1 = low ? (fa1 & 63U) : ((fc1 & 15U) | ((fa1 >> 6) << 4));
            const _Float16 c0 = static_cast<_Float16>(static_cast<float>(s0)), c1 = static_cast<_Float16>(static_cast<float>(s1));
            const _Float16 n0 = static_cast<_Float16>(-1024.0F * static_cast<float>(s0)), n1 = static_cast<_Float16>(-1024.0F * static_cast<float>(s1));
            const half2v mul0 = {c0, c0}, add0 = {n0, n0}, mul1 = {c1, c1}, add1 = {n1, n1};
            const uint32_t qs[4] = {quants.x, quants.y, quants.z, quants.w};
            const uint32_t q5[4] = {fifth.x, fifth.y, fifth.z, fifth.w};
            uint32_t lo[8], hi[8];
            const auto scaled = [&](uint32_t bytes, uint32_t sel, half2v mul, half2v add) {
                // two nibbles -> (1024 + q) as fp16 bit patterns -> sc q
                const uint32_t two = (__builtin_amdgcn_perm(0U, bytes, sel) & nibble_mask) | magic_1024;
                return __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(__builtin_bit_cast(half2v, two), mul, add));
            };
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                uint32_t w = qs[i], w4 = w >> 4;
                if (FMT == 2) {      // nibble | fifth bit << 4 per byte (sub-block 2p: bit 2p of the fifth-bit byte, 2p + 1: the next)
                    w = (w & 0x0f0f0f0fU) | (((q5[i] >> (2U * p)) & 0x01010101U) << 4);
                    w4 = (w4 & 0x0f0f0f0fU) | (((q5[i] >> (2U * p + 1U)) & 0x01010101U) << 4);
                }
                lo[2 * i] = scaled(w, 0x0c010c00U, mul0, add0); lo[2 * i + 1] = scaled(w, 0x0c030c02U, mul0, add0);
                hi[2 * i] = scaled(w4, 0x0c010c00U, mul1, add1); hi[2 * i + 1] = scaled(w4, 0x0c030c02U, mul1, add1);
            }
            uint8_t* tile_w = w_tile[p & 1U];
            *reinterpret_cast<u32x4*>(tile_w + pf_at(lrow, 2U * half)) = u32x4{lo[0], lo[1], lo[2], lo[3]};
            *reinterpret_cast<u32x4*>(tile_w + pf_at(lrow, 2U * half + 1U)) = u32x4{lo[4], lo[5], lo[6], lo[7]};
            *reinterpret_cast<u32x4*>(tile_w + pf_at(lrow, 4U + 2U * half)) = u32x4{hi[0], hi[1], hi[2], hi[3]};
            *reinterpret_cast<u32x4*>(tile_w + pf_at(lrow, 5U + 2U * half)) = u32x4{hi[4], hi[5], hi[6], hi[7]};
            if (p == 1) {
                // once per super-block, with its second step: that one is staged while the multipliers run a step without the
                // end-of-super-block work, and its results are not read before the super-block's last step
                if (half == 0) d_scale[b & 1U][lrow] = half_bits_to_float(hd.x & 0xffffU);
                // -(dmin m_j) of this super-block's eight sub-blocks: sub-blocks 8 (b % 2) .. + 8 of the group
                uint8_t* mrow = m_tile[(b >> 1) & 1U] + lrow * 64U;
                if ((b & 1U) == half) {
                    const float dm = -half_bits_to_float(hd.x >> 16);
                    uint32_t mh[4], ml[4];
#pragma unroll
                    for (int j = 0; j < 8; j += 2) {
                        float v[2];
#pragma unroll
                        for (int jj = 0; jj < 2; ++jj) {
                            const uint32_t sh = 8U * ((j + jj) & 3U);
                            const uint32_t mn = (j + jj) < 4 ? ((hd.z >> sh) & 63U) : (((hd.w >> (sh + 4U)) & 15U) | (((hd.z >> (sh + 6U)) & 3U) << 4));
                            v[jj] = dm * static_cast<float>(mn);
                        }
                        const half2v h = __builtin_convertvector(float2v{v[0], v[1]}, half2v);
                        mh[j / 2] = __builtin_bit_cast(uint32_t, h);
                        ml[j / 2] = pack_half2(v[0] - static_cast<float>(h.x), v[1] - static_cast<float>(h.y));
                    }
                    *reinterpret_cast<u32x4*>(mrow + 16U * half) = u32x4{mh[0], mh[1], mh[2], mh[3]};
                    *reinterpret_cast<u32x4*>(mrow + 32U + 16U * half) = u32x4{ml[0], ml[1], ml[2], ml[3]};
                } else if ((b & 1U) == 0 && b + 1U == blocks) {   // odd count: the last group's second super-block does not exist
                    *reinterpret_cast<u32x4*>(mrow + 16U * half) = u32x4{0U, 0U, 0U, 0U};
                    *reinterpret_cast<u32x4*>(mrow + 32U + 16U * half) = u32x4{0U, 0U, 0U, 0U};
                }
            }
        };

        // Schedule of one step (u = step % 8, super-block slot = (step / 4) % 2):
        //   [u == 0: sums copy of the next group] [token copy of step + 3] [u == 3, 7: wait for the slot staged next]
        //   stage step + 1   [u == 2, 6: fetch of the super-block two ahead into the slot just used up]
        //   wait for the token copy of step + 1, barrier.
        // Operations per step: 4 (+ 2 at u == 0, + 5 at u == 2, 6). The prologue issues the same sequence as steps
        // u = 5, 6, 7 of an iteration before the first, so the counts below hold from the first step on.
        PfRaw raw[2];
        copy_sums(0);
        fetch(0, raw[0]);
        copy_tokens(0, tok_stage[0]);
        copy_tokens(1, tok_stage[1]);
        fetch(1, raw[1]);
        copy_tokens(2, tok_stage[2]);
        // younger than the first token copy: 4 + a fetch + 4; the first fetch is older still
        if (FMT == 2) asm volatile("s_waitcnt vmcnt(14)" : "+v"(raw[0].hd), "+v"(raw[0].qs[0]), "+v"(raw[0].qs[1]), "+v"(raw[0].qs[2]), "+v"(raw[0].qs[3]), "+v"(raw[0].fifth) : : "memory");
        else asm volatile("s_waitcnt vmcnt(13)" : "+v"(raw[0].hd), "+v"(raw[0].qs[0]), "+v"(raw[0].qs[1]), "+v"(raw[0].qs[2]), "+v"(raw[0].qs[3]) : : "memory");
        stage_weights(0, 0, raw[0].hd, raw[0].qs[0], raw[0].fifth);
        pf_barrier();
        for (uint32_t s0 = 0; s0 < steps8; s0 += 8U) {
            const uint32_t b0 = s0 >> 2;
#pragma unroll
            for (uint32_t u = 0; u < 8U; ++u) {
                const uint32_t s = s0 + u;
                if (u == 0) copy_sums((s >> 3) + 1U);
                copy_tokens(s + kPfTokenAhead, tok_stage[(u + kPfTokenAhead) & 3U]);
                // the slot fetched at u == 6 of the previous iteration (u == 2 of this one): younger operations
                // 4 + 6 + 4 + (4 + a fetch) + 4 = 27 with 5 operations per fetch (4 + 4 + 4 + (4 + a fetch) + 4 = 25); Q5_K: one more
                if (FMT == 2) {
                    if (u == 3U) asm volatile("s_waitcnt vmcnt(28)" : "+v"(raw[1].hd), "+v"(raw[1].qs[0]), "+v"(raw[1].qs[1]), "+v"(raw[1].qs[2]), "+v"(raw[1].qs[3]), "+v"(raw[1].fifth) : : "memory");
                    if (u == 7U) asm volatile("s_waitcnt vmcnt(26)" : "+v"(raw[0].hd), "+v"(raw[0].qs[0]), "+v"(raw[0].qs[1]), "+v"(raw[0].qs[2]), "+v"(raw[0].qs[3]), "+v"(raw[0].fifth) : : "memory");
                } else {
                    if (u == 3U) asm volatile("s_waitcnt vmcnt(27)" : "+v"(raw[1].hd), "+v"(raw[1].qs[0]), "+v"(raw[1].qs[1]), "+v"(raw[1].qs[2]), "+v"(raw[1].qs[3]) : : "memory");
                    if (u == 7U) asm volatile("s_waitcnt vmcnt(25)" : "+v"(raw[0].hd), "+v"(raw[0].qs[0]), "+v"(raw[0].qs[1]), "+v"(raw[0].qs[2]), "+v"(raw[0].qs[3]) : : "memory");
                }
                if (s < last) stage_weights((s + 1U) >> 2, (u + 1U) & 3U, raw[((u + 1U) >> 2) & 1U].hd, raw[((u + 1U) >> 2) & 1U].qs[(u + 1U) & 3U], raw[((u + 1U) >> 2) & 1U].fifth);
                if (u == 2U) fetch(b0 + 2U, raw[0]);
                if (u == 6U) fetch(b0 + 3U, raw[1]);
                // the token copy of step s + 1 was issued in step s - 2; younger operations: a fetch in that step, then
                // the whole of steps s - 1 and s
                const uint32_t per_step[8] = {6, 4, 4 + kFetchOps, 4, 4, 4, 4 + kFetchOps, 4}, fetch_after[8] = {0, 0, kFetchOps, 0, 0, 0, kFetchOps, 0};
                switch (fetch_after[(u + 6U) & 7U] + per_step[(u + 7U) & 7U] + per_step[u]) {   // a constant once the loop is unrolled
                case 8: wait_copies<8>(); break;
                case 10: wait_copies<10>(); break;
                case 13: wait_copies<13>(); break;
                case 14: wait_copies<14>(); break;
                case 15: wait_copies<15>(); break;
                case 16: wait_copies<16>(); break;
                default: wait_copies<0>(); break;
                }
                pf_barrier();
            }
        }
        continue;
    }

    // ---- multipliers: wave (wr, wc) owns tile rows 64 wr .. + 64 (two tiles of 32 features) x tokens TS wc .. + TS
    constexpr uint32_t TT = kPfTokenTiles, TS = 32U * TT;
    floatx16 acc[TT][2], part[TT][2];              // [token tile][feature tile]
#pragma unroll
    for (int i = 0; i < static_cast<int>(TT); ++i)
#pragma unroll
        for (int n = 0; n < 2; ++n)
#pragma unroll
            for (int j = 0; j < 16; ++j) { acc[i][n][j] = 0.0F; part[i][n][j] = 0.0F; }
    const uint32_t wr = wave / (4U / TT), wc = wave % (4U / TT), l31 = lane & 31U, upper = lane >> 5;
    const uint32_t trow = (TS * wc + l31) * 128U, frow = (64U * wr + l31) * 128U, sw = (l31 >> 1) & 7U;
    uint32_t piece_at[4];
#pragma unroll
    for (uint32_t ks = 0; ks < 4U; ++ks) piece_at[ks] = ((2U * ks + upper) ^ sw) << 4;
    // token tiles of this wave that hold any row of the item (the others are neither read nor multiplied)
    const uint32_t live_tiles = count > TS * wc ? (count - TS * wc + 31U) / 32U : 0U;
    pf_barrier();
    for (uint32_t s0 = 0; s0 < steps8; s0 += 4U) {
        if (s0 >= steps) {                                    // idle steps of an odd K: keep the barrier count of the loaders
#pragma unroll
            for (uint32_t p = 0; p < 4U; ++p) pf_barrier();
            continue;
        }
#pragma unroll
        for (uint32_t p = 0; p < 4U; ++p) {
            const uint32_t s = s0 + p;
            const pf_lds* tok = tok_stage[p] + trow;
            const uint8_t* wt = w_tile[s & 1U] + frow;
            // the operands of k-step ks + 1 are read during the MFMAs of ks
            const auto k_steps = [&](auto tiles_constant) {
                constexpr uint32_t NT = decltype(tiles_constant)::value;
                half8 x[2][NT], w[2][2];
                const auto read = [&](uint32_t ks, half8 (&xs)[NT], half8 (&ws)[2]) {
#pragma unroll
                    for (uint32_t i = 0; i < NT; ++i) xs[i] = *reinterpret_cast<const __attribute__((address_space(3))) half8*>(tok + i * 32U * 128U + piece_at[ks]);
#pragma unroll
                    for (uint32_t n = 0; n < 2U; ++n) ws[n] = *reinterpret_cast<const half8*>(wt + n * 32U * 128U + piece_at[ks]);
                };
                read(0, x[0], w[0]);
                float d8[2][2];                               // Q8_0: d of the step's two blocks for the wave's two feature tiles
                if (FMT == 1) {
#pragma unroll
                    for (uint32_t g = 0; g < 2U; ++g)
#pragma unroll
                        for (uint32_t n = 0; n < 2U; ++n) d8[g][n] = d_scale[s & 1U][kPfTile * g + 64U * wr + 32U * n + l31];
                }
#pragma unroll
                for (uint32_t ks = 0; ks < 4U; ++ks) {
                    if (ks < 3U) read(ks + 1U, x[(ks + 1U) & 1U], w[(ks + 1U) & 1U]);
                    __builtin_amdgcn_sched_barrier(0);        // the reads of ks + 1 stay ahead of the MFMAs of ks
#pragma unroll
                    for (uint32_t i = 0; i < NT; ++i)
#pragma unroll
                        for (uint32_t n = 0; n < 2U; ++n) {
                            if ((FMT == 1 && (ks & 1U) == 0) || (FMT != 1 && p == 0 && ks == 0)) {   // first MFMA of a block's product: it starts from zero
                                const floatx16 zero = {0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F};
                                part[i][n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(x[ks & 1U][i], w[ks & 1U][n], zero, 0, 0, 0);
                            } else {
                                part[i][n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(x[ks & 1U][i], w[ks & 1U][n], part[i][n], 0, 0, 0);
                            }
                        }
                    __builtin_amdgcn_sched_barrier(0);
                    if (FMT == 1 && (ks & 1U)) {                  // end of a block: running sum += d * product
#pragma unroll
                        for (uint32_t i = 0; i < NT; ++i)
#pragma unroll
                            for (uint32_t n = 0; n < 2U; ++n)
#pragma unroll
                                for (int j = 0; j < 16; ++j) acc[i][n][j] = __builtin_fmaf(d8[ks >> 1][n], part[i][n][j], acc[i][n][j]);
                    }
                }
            };
            if (live_tiles >= TT) k_steps(std::integral_constant<uint32_t, TT>{});
            else if (live_tiles == 1U) k_steps(std::integral_constant<uint32_t, 1>{});
            if (FMT != 1 && p == 3U) {
                // end of a super-block: running sum += d * P (the next super-block's first MFMA starts P from zero)
                const uint32_t b = s >> 2;
                const float d[2] = {d_scale[b & 1U][64U * wr + l31], d_scale[b & 1U][64U * wr + 32U + l31]};
#pragma unroll
                for (uint32_t i = 0; i < TT; ++i)
#pragma unroll
                    for (uint32_t n = 0; n < 2U; ++n)
#pragma unroll
                        for (int j = 0; j < 16; ++j) acc[i][n][j] = __builtin_fmaf(d[n], part[i][n][j], acc[i][n][j]);   // (tiles with no live row keep P = 0)
                if (((b & 1U) || b + 1U == blocks) && live_tiles != 0 && !(MODE == 1 && a.lo_pass)) {
                    // end of a group of 16 sub-blocks: running sum += S hi * M hi + S lo * M hi + S hi * M lo
                    const uint32_t g = b >> 1;
                    const pf_lds* st = s_tile + (g & 1U) * (kPfTile * 64U) + (TS * wc + l31) * 64U + 16U * upper;
                    const uint8_t* mt = m_tile[g & 1U] + (64U * wr + l31) * 64U + 16U * upper;
                    half8 sh[TT], sl[TT], mh[2], ml[2];
#pragma unroll
                    for (uint32_t i = 0; i < TT; ++i) {
                        sh[i] = *reinterpret_cast<const __attribute__((address_space(3))) half8*>(st + i * 32U * 64U);
                        sl[i] = *reinterpret_cast<const __attribute__((address_space(3))) half8*>(st + i * 32U * 64U + 32U);
                    }
#pragma unroll
                    for (uint32_t n = 0; n < 2U; ++n) {
                        mh[n] = *reinterpret_cast<const half8*>(mt + n * 32U * 64U);
                        ml[n] = *reinterpret_cast<const half8*>(mt + n * 32U * 64U + 32U);
                    }
#pragma unroll
                    for (uint32_t i = 0; i < TT; ++i)
#pragma unroll
                        for (uint32_t n = 0; n < 2U; ++n) {
                            acc[i][n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(sh[i], mh[n], acc[i][n], 0, 0, 0);
                            acc[i][n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(sl[i], mh[n], acc[i][n], 0, 0, 0);
                            acc[i][n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(sh[i], ml[n], acc[i][n], 0, 0, 0);
                        }
                }
            }
            pf_barrier();
        }
    }

    // Result layout of a 32 x 32 tile: the lane holds feature (lane & 31); register j is token 8 (j / 4) + 4 (lane / 32) + j % 4
    const uint32_t sub_block = (m0 + 32U * wr) / 32U;         // MODE 0: the wave's 32 h values of a token are one sub-block of the down product
    uint32_t dest[TT][16];                                     // MODE 1: the assignment of every token of the lane, read ahead of all stores
    if (MODE == 1) {
#pragma unroll
        for (uint32_t i = 0; i < TT; ++i)
#pragma unroll
            for (uint32_t j = 0; j < 16U; ++j) {
                const uint32_t n = TS * wc + 32U * i + 8U * (j / 4U) + 4U * upper + (j & 3U);
                dest[i][j] = order[begin + (n < count ? n : count - 1U)];
            }
    }
#pragma unroll
    for (uint32_t i = 0; i < TT; ++i) {
#pragma unroll
        for (uint32_t j = 0; j < 16U; ++j) {
            const uint32_t n = TS * wc + 32U * i + 8U * (j / 4U) + 4U * upper + (j & 3U);
            const bool live = n < count;
            if (MODE == 0) {
                const float g = acc[i][0][j], u = acc[i][1][j];
                float gc = g, uc = u;
                swiglu_clamp(gc, uc, a.swiglu_limit);
                const float hv = (gc / (1.0F + declared_exp(-gc))) * uc;
                const _Float16 h16 = static_cast<_Float16>(hv);
                const _Float16 h16_lo = static_cast<_Float16>(hv - static_cast<float>(h16));
                float sum = live ? static_cast<float>(h16) + static_cast<float>(h16_lo) : 0.0F;
                sum += xor1_f(sum); sum += xor2_f(sum); sum += xor4_f(sum); sum += xor8_f(sum); sum += xor16_f(sum);
                if (live) {
                    a.h[static_cast<size_t>(begin + n) * a.features + m0 + 32U * wr + l31] = h16;
                    a.h_lo[static_cast<size_t>(begin + n) * a.features + m0 + 32U * wr + l31] = h16_lo;
                    if (l31 == 0) {
                        _Float16* sums = reinterpret_cast<_Float16*>(a.h_sums + static_cast<size_t>(begin + n) * pf_sum_row_bytes(a.features));
                        split_half(sum, sums[sub_block], sums[pf_sum_slots(a.features) + sub_block]);
                    }
                    if (!(finite_f(g) && finite_f(u) && finite_f(static_cast<float>(h16)))) {     // h beyond fp16 counts as non-finite
                        atomicOr(pf_status_of(a, order[begin + n]), static_cast<uint32_t>(MI355_STATUS_NONFINITE_PROJECTION));
                        atomicOr(a.job_status, static_cast<uint32_t>(MI355_STATUS_NONFINITE_PROJECTION));
                    }
                }
            } else if (live) {
                float* out = pf_rawdots_of(a, dest[i][j]) + m0 + 64U * wr + l31;
                if (a.lo_pass) {            // the second pass completes the value: the one rounding to bfloat16, if asked for, happens here
                    const float v0 = out[0] + acc[i][0][j], v1 = out[32] + acc[i][1][j];
                    out[0] = a.rawdots_bf16 ? pf_round_bf16(v0) : v0; out[32] = a.rawdots_bf16 ? pf_round_bf16(v1) : v1;
                } else { out[0] = acc[i][0][j]; out[32] = acc[i][1][j]; }
            }
        }
    }
    }   // units
}

}  // namespace strix950
