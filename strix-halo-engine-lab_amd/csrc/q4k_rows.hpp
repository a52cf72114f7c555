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
// Activation side: the 256 int8 codes of the stage's super-block of each activation row ride in the same ring slot
// (one more global_load_lds per 4 activation rows), a full stage ahead of their use; every lane reads them with broadcast
// 128-bit LDS loads. (Scalar loads of the codes were measured slower: they return out of order, so each step exposed a
// full L2 round trip.) The group deltas and sums sit one group per lane and are broadcast with v_readlane.
//
// Arithmetic per row, super-block b ascending, pair p = 0..3 (sub-blocks j = 2p: low nibbles, 2p + 1: high nibbles):
//   x_j = E_g * ((D_j * float(dot_j)) - (DM_j * float(S_g))),  D_j = d * sc_j, DM_j = dmin * m_j, g = 8 b + j
//   acc[a][p] += x_2p + x_2p+1
// and after the last super-block value = (acc_0 + acc_1) + (acc_2 + acc_3), all inside the lane. dot_j is one exact
// int32 sum of eight v_dot4_i32_i8.
// Reference arithmetic: src/cpu/core/routed_expert.cpp:73-108 == src/moe_q4k_a8_contract.cpp:126-140.
#pragma once
#include "device_math.hpp"
#include "mi355_strix.h"

namespace strix950 {

constexpr uint32_t kWaveRows = 64;
constexpr uint32_t kStageBytes = kWaveRows * 144U;   // 9,216
constexpr uint32_t kStagePieces = 9;                 // global_load_lds instructions per stage (576 pieces / 64 lanes)
// a ring slot: the stage's weights + its codes of up to nbmax (4 or 8) activation rows; a codes copy always writes four
// rows (1 KB), so only a sweep with narrow codes copies may use slot_bytes(1)
__host__ __device__ constexpr uint32_t slot_bytes(int nbmax) { return kStageBytes + 256U * static_cast<uint32_t>(nbmax); }
typedef __attribute__((address_space(3))) uint8_t lds_u8;      // ring slots are addressed in the LDS address space
template <int NA> constexpr uint32_t stage_copies() { return kStagePieces + (NA + 3) / 4; }   // copy instructions per stage


// The A8 image of a set of rows: int8 codes [width] and, per group of 32, an fp32 delta and the int32 sum of the codes.
// Image i lives at codes + (i / per_row) * codes_rs + (i % per_row) * width bytes (deltas / sums likewise, width / 32 words per
// image): per_row = 1 is one image per logical row (the input rows; every dense buffer, whose stride is then the image
// size), per_row = top_k the images of h inside strided per-row views (one per slot). With `table` set, image i is where
// table[i] points (the host executor's RowA8, src/cpu/core/routed_expert.hpp:41-45).
struct A8Image {
    const int8_t* codes;
    const float* deltas;
    const int32_t* sums;
    uint32_t width;
    uint32_t per_row;
    uint64_t codes_rs, deltas_rs, sums_rs;        // bytes between logical rows
    const mi355_row_a8* table;
    __device__ __forceinline__ void split(uint32_t i, uint32_t& q, uint32_t& s) const {
        if (per_row == 1U) { q = i; s = 0; } else { q = i / per_row; s = i - q * per_row; }
    }
    __device__ __forceinline__ const int8_t* codes_of(uint32_t i) const {
        if (table) return table[i].codes;
        uint32_t q, s;
        split(i, q, s);
        return reinterpret_cast<const int8_t*>(reinterpret_cast<const uint8_t*>(codes) + q * codes_rs + static_cast<size_t>(s) * width);
    }
    __device__ __forceinline__ const float* deltas_of(uint32_t i) const {
        if (table) return table[i].deltas;
        uint32_t q, s;
        split(i, q, s);
        return reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(deltas) + q * deltas_rs) + static_cast<size_t>(s) * (width / 32U);
    }
    __device__ __forceinline__ const int32_t* sums_of(uint32_t i) const {
        if (table) return table[i].sums;
        uint32_t q, s;
        split(i, q, s);
        return reinterpret_cast<const int32_t*>(reinterpret_cast<const uint8_t*>(sums) + q * sums_rs) + static_cast<size_t>(s) * (width / 32U);
    }
};
// one image per row, rows back to back
__host__ __device__ inline A8Image dense_image(const int8_t* codes, const float* deltas, const int32_t* sums, uint32_t width) {
    return A8Image{codes, deltas, sums, width, 1U, width, width / 8U, width / 8U, nullptr};
}

// The kernels' view of the per-row buffers: the public bundle plus what only some entry points vary. An assignment index
// i (row-major: i = row * top_k + slot, or, in the job form, the position in the job's assignment list) resolves to
// (row, slot) by place(); the per-assignment fields then sit at base + row * <field>_rs + slot * <slot extent> bytes. The
// dense bundles give <field>_rs = top_k * <slot extent>, so every address is the dense one.
struct RowsK : mi355_moe_rows {
    uint64_t slot_stride;     // floats between the slots of a row in gate_out / up_out / h_out (dense: ffn)
    A8Image in, h;            // the images of the input rows and of h
    uint64_t routes_rs, route_weights_rs, status_rs, inter_rs, rawdots_rs, base_rs;      // bytes between logical rows
    const mi355_expert_assignment* assignments;      // job form (src/cpu/core/routed_expert.hpp:47-49): item i = assignments[i]
    uint32_t top_k;
    uint32_t nonfinite_bit;   // what a non-finite gate / up / h value ORs into its row's status (8; the host executor's job: 1)
    const uint32_t* union_plan;     // verify-window form: the expert-union plan (below) names the items instead of `plan`
    uint32_t top1_form;       // a dense top-1 job whose down launch also publishes the output: combine form + 1 (0: the merge launch does)
    uint32_t* aggregate;      // optional summary word of the A8 down bindings (include/strix/moe_a8_down_contract.hpp:50-52): bit 16 beside a row's flag
    uint32_t shared_slots;    // the last shared_slots slots of a row are always-on experts: they enter the ordered combine as
                              // acc + (weight * value) in both forms (the gate scales the shared expert's output with one multiply,
                              // src/hip_shared_expert_launcher.hip:727; the sum with the routed row is one add, include/strix/moe/combine.hpp:56)
    uint32_t clean_only;      // probe form: nothing is computed or stored once the shared status word is set ("this kernel never changes
                              // status" and returns on a set one, src/hip_moe_q4k_a8_probe.hip:224-225,257-258)
    uint32_t* awords;         // a decode batch planned from early routes: one word per assignment (finished projection waves in the low
                              // half, bit 31 = non-finite projection), in place of direct updates of the status words

    __device__ __forceinline__ void place(uint32_t i, uint32_t& row, uint32_t& slot) const {
        if (assignments) { row = assignments[i].row; slot = assignments[i].slot; }
        else { row = i / top_k; slot = i - row * top_k; }
    }
    __device__ __forceinline__ uint32_t row_of(uint32_t i) const { return assignments ? assignments[i].row : i / top_k; }
    __device__ __forceinline__ const uint32_t* routes_of(uint32_t row) const {
        return reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint8_t*>(routes) + row * routes_rs);
    }
    __device__ __forceinline__ const float* route_weights_of(uint32_t row) const {
        return reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(route_weights) + row * route_weights_rs);
    }
    __device__ __forceinline__ uint32_t* status_of(uint32_t row) const {
        return reinterpret_cast<uint32_t*>(reinterpret_cast<uint8_t*>(status) + row * status_rs);
    }
    __device__ __forceinline__ const float* base_of(uint32_t row) const {
        return reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(base) + row * base_rs);
    }
    // The ordered combine of a top-1 row at the place that produced its one unweighted value (include/strix/moe/combine.hpp:36-59 with
    // one slot; product-then-add of src/ds41_expert_tp.cpp:189-199 likewise): fail closed on a flagged row, the aggregate bit for
    // a non-finite output. The caller has checked the job word.
    __device__ __forceinline__ void publish_top1(uint32_t row, uint32_t o, float raw) const {
        if (*status_of(row) & ~static_cast<uint32_t>(MI355_STATUS_AGGREGATE)) return;
        const float wt = route_weights_of(row)[0];
        const float acc = top1_form == MI355_COMBINE_FMA_SLOT_ORDER + 1U ? __builtin_fmaf(wt, raw, 0.0F) : 0.0F + wt * raw;
        const float y = base ? acc + base_of(row)[o] : acc;
        if (!finite_f(y)) atomicOr(status_of(row), static_cast<uint32_t>(MI355_STATUS_AGGREGATE));
        output[static_cast<size_t>(row) * output_stride + o] = y;
    }
    // the `hidden` unweighted outputs of assignment i
    __device__ __forceinline__ float* rawdots_of(uint32_t i, uint32_t hidden) const {
        uint32_t row, slot;
        place(i, row, slot);
        return reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(rawdots) + row * rawdots_rs) + static_cast<size_t>(slot) * hidden;
    }
    // element 0 of assignment i in one of gate_out / up_out / h_out (null stays null)
    __device__ __forceinline__ float* inter_of(float* field, uint32_t i) const {
        if (!field) return nullptr;
        uint32_t row, slot;
        place(i, row, slot);
        return reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(field) + row * inter_rs) + slot * slot_stride;
    }
    // the writable image of h of assignment i
    __device__ __forceinline__ int8_t* h_codes_of(uint32_t i) const { return const_cast<int8_t*>(h.codes_of(i)); }
    __device__ __forceinline__ float* h_deltas_of(uint32_t i) const { return const_cast<float*>(h.deltas_of(i)); }
    __device__ __forceinline__ int32_t* h_sums_of(uint32_t i) const { return const_cast<int32_t*>(h.sums_of(i)); }
};
// One work item of an expert launch: assignments [begin, end) of the plan order belong to expert e. Without a plan
// (plan == nullptr) item i is assignment i alone, its expert read from the routes (or from the job's list): the single-row
// forms of the reference entry points (include/strix/hip_moe_q4k_a8_probe.hpp:12, include/strix/hip_moe_a8_down.hpp:11-30) and
// the host executor's Job bring no plan view.
// first: the assignment at position `begin` of the plan order, plus one, when the plan's writer left it in the item's fourth
// word (the fused decode router does); 0 = look it up in the order. It spares the down + combine launch a dependent load.
struct WorkItem { uint32_t e, begin, end, first; };

// Expert-union plan of a verify window (include/strix/moe/expert_union.hpp:17-27): words {count, rows, top_k, 0}, then 128
// entries of three words {expert, slot bytes of rows 0-3, of rows 4-7}; a slot byte 0xff = that row did not choose the
// expert. Item u = entry u: its expert's weights are swept once for the rows that hold it, in ascending row order. The
// positions of such an item are (u << 8) + i, i counting the holders.
constexpr uint32_t kUnionRows = 8, kUnionTopK = 16, kUnionEntries = kUnionRows * kUnionTopK, kUnionPlanBytes = 16U + 12U * kUnionEntries;
__device__ __forceinline__ uint32_t union_held(uint32_t four_slots) {      // one bit per byte that is not 0xff, at the byte's bit 7
    const uint32_t y = ~four_slots;                                        // a byte of y is zero exactly where the slot byte is 0xff
    return (((y & 0x7f7f7f7fU) + 0x7f7f7f7fU) | y) & 0x80808080U;
}
__device__ __forceinline__ WorkItem union_item(const uint32_t* plan, uint32_t u) {
    if (u >= plan[0]) return {0U, 0U, 0U, 0U};
    const uint32_t* entry = plan + 4U + 3U * u;
    const uint32_t holders = static_cast<uint32_t>(__popc(union_held(entry[1])) + __popc(union_held(entry[2])));
    return {entry[0], u << 8, (u << 8) + holders, 0U};
}
__device__ __forceinline__ uint32_t union_assignment(const uint32_t* plan, uint32_t position) {
    const uint32_t* entry = plan + 4U + 3U * (position >> 8);
    uint32_t left = position & 255U;
    for (uint32_t row = 0; row < kUnionRows; ++row) {
        const uint32_t slot = (entry[1U + (row >> 2)] >> (8U * (row & 3U))) & 255U;
        if (slot == 255U) continue;
        if (left == 0U) return row * plan[2] + slot;
        --left;
    }
    return 0U;
}

__device__ __forceinline__ WorkItem work_item(const mi355_moe_weights& w, const RowsK& r, uint32_t items_at, uint32_t index) {
    if (r.clean_only && *r.status != 0U) return {0U, index, index, index + 1U};
    if (r.union_plan) return union_item(r.union_plan, index);
    if (r.plan) {
        const uint4 item = *reinterpret_cast<const uint4*>(r.plan + items_at + 4U * index);
        return {item.x, item.y, item.z, item.w};
    }
    uint32_t e;
    if (r.assignments) e = r.assignments[index].expert;
    else {
        uint32_t row, slot;
        r.place(index, row, slot);
        e = r.routes_of(row)[slot];
        // a route out of range: no item, and the row is flagged here as well - a caller may reach a down stage without the producer
        // that checks the routes (down_rawdots_rows flags it itself, src/hip_moe_q4k_a8_probe.hip:743)
        if (e >= w.experts) {
            atomicOr(r.status_of(row), static_cast<uint32_t>(MI355_STATUS_INVALID_ROUTE));
            if (r.aggregate) atomicOr(r.aggregate, static_cast<uint32_t>(MI355_STATUS_AGGREGATE));
        }
    }
    return {e, index, e < w.experts ? index + 1U : index, index + 1U};      // an invalid route has no item (its row is flagged)
}
__device__ __forceinline__ uint32_t ordered(const RowsK& r, uint32_t order_at, uint32_t i) {
    if (r.union_plan) return union_assignment(r.union_plan, i);
    return r.plan ? r.plan[order_at + i] : i;
}

// Per-lane source pointers of the nine pieces the lane copies in every stage. row_ptr(r) = first byte of row r (0..63).
struct StageSource {
    const uint8_t* piece[kStagePieces];
    const uint8_t* act_piece[2];              // the lane's 16 bytes of activation rows lane / 16 and 4 + lane / 16
    template <class RowPtr>
    __device__ __forceinline__ void init(RowPtr row_ptr) {
        const uint32_t lane = threadIdx.x & 63U;
#pragma unroll
        for (uint32_t i = 0; i < kStagePieces; ++i) {
            const uint32_t j = i * 64U + lane, r = __umulhi(j, 0x1C71C71DU), c = j - 9U * r;   // j / 9 exact for j < 576
            piece[i] = row_ptr(r) + 16U * c;
        }
    }
    // lane_row[h] = index (into the A8 image) of activation row 4 h + lane / 16, any valid row where that is >= NA
    template <int NA>
    __device__ __forceinline__ void init_act(const A8Image& img, const uint32_t (&lane_row)[(NA + 3) / 4]) {
        const uint32_t lane = threadIdx.x & 63U;
#pragma unroll
        for (int h = 0; h < (NA + 3) / 4; ++h)
            act_piece[h] = reinterpret_cast<const uint8_t*>(img.codes_of(lane_row[h])) + 16U * (lane & 15U);
    }
    // start the copy of the next super-block of all 64 rows (and of the activation rows' codes) into one ring slot,
    // then step to the block after it
    // A codes copy moves four activation rows (1 KB: lanes 16 a .. 16 a + 15 move row a). NARROW (NA == 1 only): just the
    // first sixteen lanes take part, so the slot ends 256 bytes after the weights (slot_bytes(1)) instead of 1 KB after them.
    template <int NA, bool NARROW = false>
    __device__ __forceinline__ void start(lds_u8* slot) {
        static_assert(!NARROW || NA == 1, "a narrow codes copy serves one activation row");
#pragma unroll
        for (uint32_t i = 0; i < kStagePieces; ++i) {
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)piece[i],
                                             (__attribute__((address_space(3))) void*)(slot + 1024U * i), 16, 0, 0);
            piece[i] += 144;
        }
#pragma unroll
        for (int h = 0; h < (NA + 3) / 4; ++h) {
            if (!NARROW || (threadIdx.x & 63U) < 16U)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)act_piece[h],
                                                 (__attribute__((address_space(3))) void*)(slot + kStageBytes + 1024U * h), 16, 0, 0);
            act_piece[h] += 256;
        }
    }
};

// s_waitcnt vmcnt(N) lgkmcnt(0): at most N vector memory operations (here: stage copies, PER per stage) still outstanding, and
// every LDS read of this wave returned - the copy that follows overwrites a slot this wave has read, and a copy's data is
// written to LDS when it arrives, whatever reads of the slot are still queued there.
template <int N>
__device__ __forceinline__ void wait_copies() {
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (0 << 8));
}
template <int PER>
__device__ __forceinline__ void wait_stages_ahead(uint32_t ahead) {   // ahead = stages started after the one needed
    if (ahead == 0) wait_copies<0>();
    else if (ahead == 1) wait_copies<PER>();
    else if (ahead == 2) wait_copies<2 * PER>();
    else wait_copies<3 * PER>();
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

// Uniform view of the NA activation rows of one sweep (row bases, wave-uniform).
template <int NA>
struct ActRows {
    A8Image img;
    uint32_t lane_row[(NA + 3) / 4];           // per lane: image row of activation row 4 h + lane / 16 (see StageSource::init_act)
    const float* deltas[NA];
    const int32_t* sums[NA];
    uint32_t groups;                           // per activation row
    // row[a]: image row of activation row a (any lane's value is taken); lane_rows: the per-lane rows for the code copies
    __device__ __forceinline__ ActRows(const A8Image& img, const uint32_t (&row)[NA], const uint32_t (&lane_rows)[(NA + 3) / 4])
        : img(img), groups(img.width / 32U) {
#pragma unroll
        for (int h = 0; h < (NA + 3) / 4; ++h) lane_row[h] = lane_rows[h];
#pragma unroll
        for (int a = 0; a < NA; ++a) {
            const uint32_t r = __builtin_amdgcn_readfirstlane(row[a]);
            deltas[a] = img.deltas_of(r);
            sums[a] = img.sums_of(r);
        }
    }
};

__device__ __forceinline__ float lane_value(float v, uint32_t lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), static_cast<int>(lane)));
}

// One super-block (index kb along K) of the lane's row against the NA activation rows, both from ring slot `slot`.
// vd / vf: the activation rows' group deltas / sums, group 8 (kb % 8) + j in lane 8 (kb % 8) + j.
template <int NA>
__device__ __forceinline__ void block_compute(const lds_u8* slot, uint32_t kb, const float (&vd)[NA], const float (&vf)[NA],
                                              float (&acc)[NA][4]) {
    typedef const __attribute__((address_space(3))) u32x4 lds_u32x4;
    lds_u32x4* blk = (lds_u32x4*)(slot + (threadIdx.x & 63U) * 144U);
    const u32x4 hd = blk[0];
    u32x4 q[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) q[i] = blk[1 + i];
    const float d = half_bits_to_float(hd.x & 0xffffU), dm = half_bits_to_float(hd.x >> 16);
    uint32_t sc[8], mn[8];
    q4k_factors<0>(hd, sc[0], mn[0]); q4k_factors<1>(hd, sc[1], mn[1]); q4k_factors<2>(hd, sc[2], mn[2]); q4k_factors<3>(hd, sc[3], mn[3]);
    q4k_factors<4>(hd, sc[4], mn[4]); q4k_factors<5>(hd, sc[5], mn[5]); q4k_factors<6>(hd, sc[6], mn[6]); q4k_factors<7>(hd, sc[7], mn[7]);
    float D[8], M[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        D[j] = d * static_cast<float>(sc[j]);
        M[j] = dm * static_cast<float>(mn[j]);
    }
    const uint32_t g0 = (kb & 7U) * 8U;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const uint32_t w[8] = {q[2 * p].x, q[2 * p].y, q[2 * p].z, q[2 * p].w, q[2 * p + 1].x, q[2 * p + 1].y, q[2 * p + 1].z, q[2 * p + 1].w};
        int lo[8], hi[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            lo[k] = static_cast<int>(w[k] & 0x0f0f0f0fU);
            hi[k] = static_cast<int>((w[k] >> 4) & 0x0f0f0f0fU);
        }
#pragma unroll
        for (int a = 0; a < NA; ++a) {
            lds_u32x4* codes = (lds_u32x4*)(slot + kStageBytes + 256U * a + 64U * p);
            const u32x4 c0 = codes[0], c1 = codes[1], c2 = codes[2], c3 = codes[3];
            const uint32_t c[16] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w, c2.x, c2.y, c2.z, c2.w, c3.x, c3.y, c3.z, c3.w};
            int dot0 = 0, dot1 = 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                dot0 = __builtin_amdgcn_sdot4(lo[k], static_cast<int>(c[k]), dot0, false);
                dot1 = __builtin_amdgcn_sdot4(hi[k], static_cast<int>(c[8 + k]), dot1, false);
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

// Whole sweep: K = blocks super-blocks of the 64 rows described by `source` against the NA rows of `act`.
// value[a] = the lane's row against activation row a. `slots` are DEPTH separate LDS buffers of slot_bytes().
// On entry nothing is in flight; on exit every copy has landed and been consumed.
template <int NA, int DEPTH, bool NARROW = false>
__device__ __forceinline__ void sweep_rows(lds_u8* const (&slots)[DEPTH], StageSource source, uint32_t blocks,
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
    source.init_act<NA>(act.img, act.lane_row);
#pragma unroll
    for (int s = 0; s < DEPTH - 1; ++s)
        if (static_cast<uint32_t>(s) < blocks) source.start<NA, NARROW>(slots[s]);
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
                wait_stages_ahead<stage_copies<NA>()>(last - 1U - b);
                if (b + DEPTH - 1U < blocks) source.start<NA, NARROW>(slots[(s + DEPTH - 1) % DEPTH]);
                block_compute<NA>(slots[s], b, vd, vf, acc);
            }
        }
    }
#pragma unroll
    for (int a = 0; a < NA; ++a) value[a] = (acc[a][0] + acc[a][1]) + (acc[a][2] + acc[a][3]);
}

}  // namespace strix950
