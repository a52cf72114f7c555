// The reference's A8 request / bindings boundary on this library's kernels: host admission (pure: no allocation, no device
// call, no buffer touched) and the single-row ("C1") entry points with up to 16 logical rows.
//   Request / Shape / Bindings / validate     include/strix/moe_q4k_a8_contract.hpp:104-122, src/moe_q4k_a8_contract.cpp:343-372
//   enqueue_probe                             include/strix/hip_moe_q4k_a8_probe.hpp:8-12
//   DownRequest / DownBindings / validate_down include/strix/moe_a8_down_contract.hpp:40-54, src/moe_a8_down_contract.cpp:53-82
//   enqueue_down_activation_quantize / enqueue_down_rawdots (+ SlotMergeTail)   include/strix/hip_moe_a8_down.hpp:11-30
// Differences from the reference, all widening: the geometry caps (hidden 2560, rows 1536, experts 512) are this library's
// (hidden <= 16384, intermediate <= 16384, experts <= 1024, top_k <= 16), fp16 input is a third input kind, and
// shape.logical_rows may be 1..16 with the per-row views holding that many contiguous single-row extents (the reference's
// union form without its plan view: an expert chosen by two rows is simply read twice).
// Status words are the caller's and sticky: nothing here clears them, bits are OR-ed in.
//   union rows form (a verify window of R <= 8 rows reads each distinct expert once): the plan of
//   include/strix/moe/expert_union.hpp:17-57 built on the device, validate_union (src/moe_q4k_a8_contract.cpp:373-405),
//   validate_down_union (src/moe_a8_down_contract.cpp:83-113), enqueue_probe_union / enqueue_down_*_union
//   (src/hip_moe_q4k_a8_probe.hip:1172-1221). The items of the expert sweeps are then the plan's entries (q4k_rows.hpp).
#pragma once

namespace strix950 {

constexpr uint32_t kA8MaxHidden = 16384, kA8MaxIntermediate = 16384, kA8MaxLogicalRows = 16;

inline bool a8_identity_matches(const char* given, uint32_t type, int down) {
    const char* mine = mi355_numerical_identity(type, down);
    return given != nullptr && mine[0] != 0 && std::strcmp(given, mine) == 0;
}
inline bool a8_overlap(const mi355_device_bytes& x, const mi355_device_bytes& y) {
    return !(x.address + x.bytes <= y.address || y.address + y.bytes <= x.address);
}
inline bool a8_clamp_ok(float limit) { return limit == INFINITY || (std::isfinite(limit) && limit > 0.0F); }

// gate / up row bytes per 256 weights (src/moe_q4k_a8_contract.cpp:352-354: Q4_K 144, Q5_K 176)
inline uint64_t a8_gate_block_bytes(uint32_t type) { return type == MI355_TYPE_Q5_K ? 176U : 144U; }

int32_t a8_validate(const mi355_a8_request* q, const mi355_a8_bindings* b) {
    STRIX_REQUIRE(q && b, "A8 probe: null request or bindings");
    STRIX_REQUIRE(q->enabled && a8_identity_matches(q->approved_numerical_identity, q->gate_type, 0),
                  "A8 probe requires explicit matching numerical identity approval (mi355_numerical_identity(gate_type, 0))");
    const mi355_a8_shape& s = q->shape;
    STRIX_REQUIRE(s.hidden >= 256 && s.hidden <= kA8MaxHidden && s.hidden % 256U == 0 && s.rows > 0 && s.rows <= kA8MaxIntermediate &&
                  s.rows % 32U == 0 && s.experts > 0 && s.experts <= kRouteMaxExperts && s.top_k > 0 && s.top_k <= kRouteMaxTopK &&
                  s.logical_rows >= 1 && s.logical_rows <= kA8MaxLogicalRows,
                  "A8 probe admits hidden % 256 (<= 16384), rows % 32 (<= 16384), experts <= 1024, top_k <= 16, logical_rows 1..16 only");
    STRIX_REQUIRE(q->input <= MI355_INPUT_BF16, "A8 probe: input storage unsupported");
    STRIX_REQUIRE(q->gate_type == q->up_type && !q->fused_gate_up && (q->gate_type == MI355_TYPE_Q4_K || q->gate_type == MI355_TYPE_Q5_K),
                  "A8 probe requires separate matching type 12 or type 13 gate / up tensors");
    STRIX_REQUIRE(q->swiglu_limit == INFINITY, "A8 probe: a finite SwiGLU clamp belongs to the down producer (DownRequest), not to the projection");
    const uint64_t R = s.logical_rows;
    const uint64_t weight_bytes = static_cast<uint64_t>(s.experts) * s.rows * (s.hidden / 256U) * a8_gate_block_bytes(q->gate_type);
    const mi355_device_bytes views[9] = {b->input, b->gate, b->up, b->routes, b->codes, b->deltas, b->sums, b->status, b->output};
    const uint64_t required[9] = {R * s.hidden * (q->input == MI355_INPUT_F32 ? 4U : 2U), weight_bytes, weight_bytes, R * s.top_k * 4ULL,
                                  R * s.hidden, R * (s.hidden / 32U) * 4ULL, R * (s.hidden / 32U) * 4ULL, 4,
                                  R * s.top_k * 2ULL * s.rows * 4ULL};
    for (size_t i = 0; i < 9; ++i) {
        STRIX_REQUIRE(views[i].address != 0 && views[i].address % 16U == 0 && views[i].bytes == required[i] &&
                      views[i].bytes <= UINTPTR_MAX - views[i].address, "A8 probe device view address / alignment / exact byte size invalid");
        // every mutable view (codes, deltas, sums, status, output) is disjoint from every other view; gate and up are separate
        for (size_t j = 0; j < i; ++j)
            if (i >= 4 || (i == 2 && j == 1))
                STRIX_REQUIRE(!a8_overlap(views[i], views[j]), "A8 probe mutable views and separate gate / up must not overlap");
    }
    return MI355_OK;
}

inline uint64_t a8_down_row_bytes(uint32_t type, uint32_t intermediate) {        // src/moe_a8_down_contract.cpp:47-52
    if (type == MI355_TYPE_Q4_K) return static_cast<uint64_t>(intermediate / 256U) * 144U;
    if (type == MI355_TYPE_Q6_K) return static_cast<uint64_t>(intermediate / 256U) * 210U;
    return static_cast<uint64_t>(intermediate / 32U) * (type == MI355_TYPE_Q5_1 ? 24U : 34U);
}

int32_t a8_validate_down(const mi355_a8_down_request* q, const mi355_a8_down_bindings* b, uint32_t logical_rows) {
    STRIX_REQUIRE(q && b, "A8 down: null request or bindings");
    if (!(q->weight_type == MI355_TYPE_Q4_K || q->weight_type == MI355_TYPE_Q6_K || q->weight_type == MI355_TYPE_Q5_1 || q->weight_type == MI355_TYPE_Q8_0))
        return fail(MI355_E_UNSUPPORTED, "A8 down weights must be Q5_1 (7), Q8_0 (8), Q4_K (12) or Q6_K (14)");
    STRIX_REQUIRE(q->enabled && a8_identity_matches(q->approved_numerical_identity, q->weight_type, 1),
                  "A8 down requires explicit matching numerical identity (mi355_numerical_identity(weight_type, 1))");
    STRIX_REQUIRE(a8_clamp_ok(q->swiglu_limit), "A8 down SwiGLU clamp limit must be +infinity (none) or finite positive");
    const mi355_a8_down_shape& s = q->shape;
    const bool kq = q->weight_type == MI355_TYPE_Q4_K || q->weight_type == MI355_TYPE_Q6_K;
    STRIX_REQUIRE(s.hidden > 0 && s.hidden <= kA8MaxHidden && s.hidden % 64U == 0 && s.intermediate > 0 && s.intermediate <= kA8MaxIntermediate &&
                  s.intermediate % (kq ? 256U : 128U) == 0 && s.experts > 0 && s.experts <= kRouteMaxExperts && s.top_k > 0 && s.top_k <= kRouteMaxTopK &&
                  logical_rows >= 1 && logical_rows <= kA8MaxLogicalRows,
                  "A8 down admits hidden % 64, intermediate % 128 (K-quant: % 256), experts <= 1024, top_k <= 16, rows 1..16 only");
    const uint64_t R = logical_rows, groups = static_cast<uint64_t>(s.top_k) * (s.intermediate / 32U);
    const mi355_device_bytes views[9] = {b->intermediates, b->weights, b->routes, b->codes, b->deltas, b->sums, b->rawdots, b->status, b->aggregate_status};
    const uint64_t bytes[9] = {R * s.top_k * 2ULL * s.intermediate * 4ULL,
                               static_cast<uint64_t>(s.experts) * s.hidden * a8_down_row_bytes(q->weight_type, s.intermediate),
                               R * s.top_k * 4ULL, R * s.top_k * static_cast<uint64_t>(s.intermediate), R * groups * 4ULL, R * groups * 4ULL,
                               R * s.top_k * static_cast<uint64_t>(s.hidden) * 4ULL, 4, 4};
    // the weight tensor starts on 16 bytes in every class (the reference asks that of Q4_K only and 2 bytes of the others,
    // src/moe_a8_down_contract.cpp:72-73; the kernels here read words and quads relative to the tensor's start)
    const unsigned align[9] = {16, 16, 4, 16, 16, 16, 16, 4, 4};
    for (size_t i = 0; i < 9; ++i) {
        if (i == 8 && views[i].address == 0 && views[i].bytes == 0) continue;     // the aggregate word is optional
        STRIX_REQUIRE(views[i].address != 0 && views[i].address % align[i] == 0 && views[i].bytes == bytes[i] &&
                      bytes[i] <= UINTPTR_MAX - views[i].address, "A8 down view alignment / address / exact extent invalid");
        for (size_t j = 0; j < i; ++j) STRIX_REQUIRE(!a8_overlap(views[i], views[j]), "A8 down views must be disjoint");
    }
    return MI355_OK;
}

// ---------------------------------------------------------------------------------------------------------- kernels
// The union plan of R x top_k routes, built by the first two wavefronts of one 256-thread workgroup, thread t = assignment t = (row t / top_k, slot t % top_k).
// An assignment is a "first" when no earlier assignment names its expert; the firsts, in assignment order, are the entries.
// An expert id >= experts or an expert named twice by one row sets MI355_STATUS_INVALID_ROUTE and leaves count = 0 (no sweep
// runs). All 128 entries are written: the unused ones hold expert 0 and 0xff slots.
__device__ __forceinline__ void a8_union_plan_block(const uint32_t* routes, uint32_t rows, uint32_t top_k, uint32_t experts, uint32_t* plan, uint32_t* status) {
    __shared__ __attribute__((aligned(16))) uint32_t expert_of[kUnionEntries];
    __shared__ uint32_t entry_of_first[kUnionEntries], entry_expert[kUnionEntries];
    __shared__ uint8_t entry_slots[kUnionEntries][kUnionRows];
    __shared__ uint32_t firsts_in_wave0, invalid;
    const uint32_t t = threadIdx.x, n = rows * top_k, lane = t & 63U;
    const bool mine = t < kUnionEntries;                   // thread t of the first two wavefronts = assignment t = entry t
    uint32_t e = 0xffffffffU;
    if (mine) {
        if (t == 0) invalid = 0;
        entry_expert[t] = 0;
        reinterpret_cast<uint32_t*>(entry_slots[t])[0] = 0xffffffffU;
        reinterpret_cast<uint32_t*>(entry_slots[t])[1] = 0xffffffffU;
        if (t < n) e = routes[t];
        expert_of[t] = e;
    }
    __syncthreads();
    uint32_t first = t, before = 0;
    bool is_first = false;
    if (mine) {
        bool bad = false;
        if (t < n) {
            // the earliest assignment with this expert: every lane reads every word (broadcast reads, no early exit to wait for)
            typedef const uint32_t u32x4_s __attribute__((ext_vector_type(4)));
            const u32x4_s* four = reinterpret_cast<const u32x4_s*>(expert_of);
#pragma unroll 8
            for (uint32_t a = 0; a < (n + 3U) / 4U; ++a) {
                const auto q = four[a];
                const uint32_t hit = q.x == e ? 4U * a : q.y == e ? 4U * a + 1U : q.z == e ? 4U * a + 2U : q.w == e ? 4U * a + 3U : 0xffffffffU;
                first = hit < first ? hit : first;
            }
            bad = e >= experts || (first != t && first >= t - t % top_k);
        }
        is_first = t < n && first == t;
        const uint64_t firsts = __ballot(is_first);
        if (t == 0) firsts_in_wave0 = static_cast<uint32_t>(__popcll(firsts));
        if (__ballot(bad) != 0 && lane == 0) invalid = 1;
        before = static_cast<uint32_t>(__popcll(firsts & ((1ULL << lane) - 1ULL)));
    }
    __syncthreads();
    if (mine) {
        before += t >= 64U ? firsts_in_wave0 : 0U;
        if (is_first) { entry_of_first[t] = before; entry_expert[before] = e; }
    }
    __syncthreads();
    if (mine && t < n) entry_slots[entry_of_first[first]][t / top_k] = static_cast<uint8_t>(t % top_k);
    __syncthreads();
    if (!mine) return;
    if (t == kUnionEntries - 1U) {         // (the last thread of the second wave knows the number of entries)
        const uint32_t count = before + (is_first ? 1U : 0U);
        plan[0] = invalid ? 0U : count; plan[1] = rows; plan[2] = top_k; plan[3] = 0U;
        if (invalid) atomicOr(status, static_cast<uint32_t>(MI355_STATUS_INVALID_ROUTE));
    }
    uint32_t* entry = plan + 4U + 3U * t;
    entry[0] = entry_expert[t];
    entry[1] = reinterpret_cast<const uint32_t*>(entry_slots[t])[0];
    entry[2] = reinterpret_cast<const uint32_t*>(entry_slots[t])[1];
}

// Route check + A8 image of the input rows of the probe (src/hip_moe_q4k_a8_probe.hip:41-90: validation and quantizer of one
// row; here blockIdx.y = logical row). Block x quantises 8 groups of 32; block (0, row) also checks the row's routes.
template <int KIND>
__global__ __launch_bounds__(256) void a8_probe_prologue_kernel(const uint8_t* x, uint32_t hidden, const uint32_t* routes, uint32_t experts,
                                                                uint32_t top_k, int8_t* codes, float* deltas, int32_t* sums, uint32_t* status,
                                                                uint32_t* union_plan, uint32_t union_top_k) {
    const uint32_t r = blockIdx.y, groups = hidden / 32U, g = blockIdx.x * 8U + (threadIdx.x >> 5), j = threadIdx.x & 31U;
    // the union rows form: one more block per launch builds the plan beside the quantiser's blocks
    if (union_plan && blockIdx.x == gridDim.x - 1U) {
        if (r == 0) a8_union_plan_block(routes, gridDim.y, union_top_k, experts, union_plan, status);
        return;
    }
    if (blockIdx.x == 0 && threadIdx.x < top_k && routes[r * top_k + threadIdx.x] >= experts) atomicOr(status, static_cast<uint32_t>(MI355_STATUS_INVALID_ROUTE));
    if (g >= groups) return;
    // the probe contract's quantiser ("g32-sym127-zero1-finite-noflush", src/moe_q4k_a8_contract.cpp:67-91): delta = amax / 127
    // with no tiny-group rule; a non-finite value is flagged and taken as 0, a delta that underflows to 0 is flagged and taken as 1
    float v = load_activation<KIND>(x + static_cast<size_t>(r) * hidden * (KIND == 0 ? 4U : 2U), g * 32U + j);
    const int bad = or32_i(finite_f(v) ? 0 : 1);
    if (!finite_f(v)) v = 0.0F;
    const float amax = max32(__builtin_fabsf(v));
    float delta = amax == 0.0F ? 1.0F : amax / 127.0F;
    const bool underflow = !(delta > 0.0F) || !finite_f(delta);
    if (underflow) delta = 1.0F;
    const int code = a8_code(v, delta, false);
    const int sum = sum32_i(code);
    codes[static_cast<size_t>(r) * hidden + g * 32U + j] = static_cast<int8_t>(code);
    if (j == 0) {
        deltas[static_cast<size_t>(r) * groups + g] = delta;
        sums[static_cast<size_t>(r) * groups + g] = sum;
        if (bad) atomicOr(status, static_cast<uint32_t>(MI355_STATUS_NONFINITE_ACTIVATION));
        if (underflow) atomicOr(status, static_cast<uint32_t>(MI355_STATUS_INVALID_DELTA));
    }
}

// One serial row's prologue in one workgroup, with the reference's store rules (src/hip_moe_q4k_a8_probe.hip:47-90,187-199):
//   SERIAL: zero clear[0 .. clear_words), check the routes (an index out of range or a non-finite route weight: bit 1), quantise
//           unless a route failed, and OVERWRITE the status word with route bits | quantiser bits;
//   else:   the pair validate_routes + quantize: OR bit 1 for an index out of range (route weights are not looked at), quantise only
//           when the status word is still zero after that, OR the quantiser's bits in.
// The quantiser stages codes / deltas / sums in LDS and stores them only when the whole row is clean: a flagged step leaves the
// image of the previous step in place.
template <int KIND, bool SERIAL>
__global__ __launch_bounds__(1024) void a8_serial_prologue_kernel(const uint8_t* x, const uint32_t* routes, const float* route_weights, float* clear,
                                                                  uint32_t clear_words, uint32_t hidden, uint32_t top_k, uint32_t experts,
                                                                  int8_t* codes, float* deltas, int32_t* sums, uint32_t* status) {
    __shared__ __attribute__((aligned(16))) int8_t local_codes[kA8MaxHidden];
    __shared__ __attribute__((aligned(16))) float local_deltas[kA8MaxHidden / 32U];
    __shared__ __attribute__((aligned(16))) int32_t local_sums[kA8MaxHidden / 32U];
    __shared__ uint32_t route_bits, bad_bits, initial;
    const uint32_t t = threadIdx.x, groups = hidden / 32U;
    if (t == 0) { route_bits = 0; bad_bits = 0; initial = SERIAL ? 0U : *status; }
    if (SERIAL) for (uint32_t i = t; i < clear_words; i += 1024U) clear[i] = 0.0F;
    __syncthreads();
    if (t < top_k && (routes[t] >= experts || (SERIAL && !finite_f(route_weights[t])))) atomicOr(&route_bits, static_cast<uint32_t>(MI355_STATUS_INVALID_ROUTE));
    __syncthreads();
    const uint32_t before = initial | route_bits;
    if (!SERIAL && t == 0 && route_bits) atomicOr(status, route_bits);
    if (before != 0U) {                                      // the quantiser is skipped: nothing stored
        if (SERIAL && t == 0) *status = route_bits;
        return;
    }
    for (uint32_t g = t >> 5; g < groups; g += 32U) {
        const uint32_t i = g * 32U + (t & 31U);
        float v = load_activation<KIND>(x, i);
        const int bad = or32_i(finite_f(v) ? 0 : 1);
        if (!finite_f(v)) v = 0.0F;
        const float amax = max32(__builtin_fabsf(v));
        float delta = amax == 0.0F ? 1.0F : amax / 127.0F;
        const bool underflow = !(delta > 0.0F) || !finite_f(delta);
        if (underflow) delta = 1.0F;
        const int code = a8_code(v, delta, false);
        const int sum = sum32_i(code);
        local_codes[i] = static_cast<int8_t>(code);
        if ((t & 31U) == 0) {
            local_deltas[g] = delta; local_sums[g] = sum;
            if (bad) atomicOr(&bad_bits, static_cast<uint32_t>(MI355_STATUS_NONFINITE_ACTIVATION));
            if (underflow) atomicOr(&bad_bits, static_cast<uint32_t>(MI355_STATUS_INVALID_DELTA));
        }
    }
    __syncthreads();
    const uint32_t bad = bad_bits;
    if (bad == 0U) {
        for (uint32_t i = t; i < hidden / 16U; i += 1024U) reinterpret_cast<u32x4*>(codes)[i] = reinterpret_cast<const u32x4*>(local_codes)[i];
        for (uint32_t i = t; i < groups; i += 1024U) { deltas[i] = local_deltas[i]; sums[i] = local_sums[i]; }
    }
    if (t == 0) {
        if (SERIAL) *status = bad;
        else if (bad) atomicOr(status, bad);
    }
}

// The down producer (src/hip_moe_q4k_a8_probe.hip:594-621): intermediates hold, per assignment, [gate I | up I]; h replaces the
// gate half, its A8 image goes to codes / deltas / sums [assignment][I]. One half-wave per group of 32.
__global__ __launch_bounds__(256) void a8_down_activation_kernel(float* intermediates, const uint32_t* routes, uint32_t experts, uint32_t width,
                                                                 uint32_t exp_kind, float limit, int8_t* codes, float* deltas, int32_t* sums,
                                                                 uint32_t* status, uint32_t* aggregate) {
    const uint32_t a = blockIdx.y, groups = width / 32U, grp = blockIdx.x * 8U + (threadIdx.x >> 5), l = threadIdx.x & 31U;
    if (grp >= groups) return;
    if (routes[a] >= experts) {
        if (l == 0) { atomicOr(status, static_cast<uint32_t>(MI355_STATUS_INVALID_ROUTE)); if (aggregate) atomicOr(aggregate, static_cast<uint32_t>(MI355_STATUS_AGGREGATE)); }
        return;
    }
    const size_t at = static_cast<size_t>(a) * 2U * width + grp * 32U + l;
    const float g = intermediates[at], u = intermediates[at + width];
    float gc = g, uc = u;
    swiglu_clamp(gc, uc, limit);
    const float hv = (gc / (1.0F + exp_of(exp_kind, -gc))) * uc;
    if (or32_i((finite_f(g) && finite_f(u) && finite_f(hv)) ? 0 : 1)) {
        if (l == 0) { atomicOr(status, static_cast<uint32_t>(MI355_STATUS_NONFINITE_PROJECTION)); if (aggregate) atomicOr(aggregate, static_cast<uint32_t>(MI355_STATUS_AGGREGATE)); }
        return;
    }
    const float amax = max32(__builtin_fabsf(hv));
    const bool tiny = amax > 0.0F && amax < 0x1p-119F;
    const float dl = (amax == 0.0F || tiny) ? 1.0F : amax / 127.0F;
    const int code = a8_code(hv, dl, tiny);
    const int sum = sum32_i(code);
    intermediates[at] = hv;
    codes[static_cast<size_t>(a) * width + grp * 32U + l] = static_cast<int8_t>(code);
    if (l == 0) { deltas[static_cast<size_t>(a) * groups + grp] = dl; sums[static_cast<size_t>(a) * groups + grp] = sum; }
}

// Expert-slot merge, commit and first-error record of one row after its rawdots (include/strix/moe_slot_merge.hpp:47-55,
// src/hip_moe_q4k_a8_probe.hip:825-897): per output +0, then fma(route_weight[slot], rawdots[slot][o], acc) in slot order (nothing
// is written when the status was already set or a route is invalid); a value at or above the commit threshold (bf16
// commit: 0x7f7f8000, the finite values that round to bf16 infinity included) fails the whole step: status |= 8 and no output
// is committed; the record keeps the first non-zero status of the stream. One 1024-thread workgroup.
struct SlotMergeArgs {
    const float* rawdots; const uint32_t* routes; uint32_t* status; uint32_t hidden, experts, top_k;
    const float* route_weights; float* accumulation; void* output; uint32_t output_bf16, bf16_commit; uint32_t* record; uint32_t domain;
};
__global__ __launch_bounds__(1024) void a8_slot_merge_kernel(SlotMergeArgs t) {
    __shared__ uint32_t flagged, invalid;
    if (threadIdx.x == 0) { flagged = 0; invalid = 0; }
    __syncthreads();
    // an invalid route fails the step whatever ran before: the rawdots launch in front of this one flags it as well, but a status
    // word cleared in between must not let a stale accumulation through (src/hip_moe_q4k_a8_probe.hip:743)
    if (threadIdx.x < t.top_k && t.routes[threadIdx.x] >= t.experts) invalid = 1;
    __syncthreads();
    if (threadIdx.x == 0 && invalid) atomicOr(t.status, static_cast<uint32_t>(MI355_STATUS_INVALID_ROUTE));
    const uint32_t initial = *t.status | (invalid ? static_cast<uint32_t>(MI355_STATUS_INVALID_ROUTE) : 0U);
    if (initial == 0U) {
        const bool written = invalid == 0;
        for (uint32_t o = threadIdx.x; o < t.hidden; o += 1024U) {
            float current = 0.0F;
            if (written) {
                for (uint32_t k = 0; k < t.top_k; ++k) current = __builtin_fmaf(t.route_weights[k], t.rawdots[static_cast<size_t>(k) * t.hidden + o], current);
                t.accumulation[o] = current;
            }
            const float value = written ? current : t.accumulation[o];
            if ((b_of(value) & 0x7fffffffU) >= (t.bf16_commit ? 0x7f7f8000U : 0x7f800000U)) flagged = 1;
        }
    }
    __syncthreads();
    const uint32_t final_status = initial | (flagged ? 8U : 0U);
    if (final_status == 0U)
        for (uint32_t o = threadIdx.x; o < t.hidden; o += 1024U) {
            const uint32_t bits = b_of(t.accumulation[o]);
            if (t.output_bf16) static_cast<unsigned short*>(t.output)[o] = static_cast<unsigned short>((bits + 0x7fffU + ((bits >> 16) & 1U)) >> 16);
            else static_cast<float*>(t.output)[o] = f_of(bits);
        }
    if (threadIdx.x == 0) {
        if (flagged) atomicOr(t.status, 8U);
        // DeferredMoeFirstError {domain, bits}: the first non-zero status of the stream stays (include/strix/deferred_moe_status.hpp:19-26)
        if (final_status != 0U && t.record[0] == 0U) { t.record[1] = final_status; t.record[0] = t.domain; }
    }
}

// ---------------------------------------------------------------------------------------------------------- union rows
inline bool a8_union_admits(uint32_t rows, uint32_t top_k) { return rows >= 1U && rows <= kUnionRows && top_k >= 1U && top_k <= kUnionTopK; }
inline int32_t a8_union_plan_view(const mi355_device_bytes& plan) {
    STRIX_REQUIRE(plan.address != 0 && plan.address % 16U == 0 && plan.bytes == kUnionPlanBytes && plan.bytes <= UINTPTR_MAX - plan.address,
                  "A8 union plan view invalid: 16-byte aligned, exactly 1552 bytes");
    return MI355_OK;
}

int32_t a8_validate_union(const mi355_a8_request* q, const mi355_a8_bindings* b, const mi355_device_bytes& plan) {
    STRIX_REQUIRE(q && b, "A8 union probe: null request or bindings");
    const mi355_a8_shape& s = q->shape;
    STRIX_REQUIRE(a8_union_admits(s.logical_rows, s.top_k) && q->gate_type == MI355_TYPE_Q4_K, "A8 union rows admit R <= 8, K <= 16 and Q4_K gate / up only");
    // every row slice is a single-row bundle of its own: with R > 1 the per-row extents keep the slices on 16 bytes
    STRIX_REQUIRE(s.logical_rows == 1U || (s.top_k * 4U) % 16U == 0, "A8 union per-row views: every row slice must start on 16 bytes (top_k % 4 == 0 for R > 1)");
    if (const int32_t rc = a8_validate(q, b)) return rc;
    if (const int32_t rc = a8_union_plan_view(plan)) return rc;
    const mi355_device_bytes views[9] = {b->input, b->gate, b->up, b->routes, b->codes, b->deltas, b->sums, b->status, b->output};
    for (const mi355_device_bytes& v : views) STRIX_REQUIRE(!a8_overlap(plan, v), "A8 union plan must not overlap any other view");
    return MI355_OK;
}

int32_t a8_validate_down_union(const mi355_a8_down_request* q, const mi355_a8_down_bindings* b, uint32_t rows, const mi355_device_bytes& plan) {
    STRIX_REQUIRE(q && b, "A8 down union: null request or bindings");
    STRIX_REQUIRE(a8_union_admits(rows, q->shape.top_k) && (q->weight_type == MI355_TYPE_Q4_K || q->weight_type == MI355_TYPE_Q6_K),
                  "A8 down union rows admit R <= 8, K <= 16 and the K-quant class (Q4_K / Q6_K) only");
    if (const int32_t rc = a8_validate_down(q, b, rows)) return rc;
    if (const int32_t rc = a8_union_plan_view(plan)) return rc;
    const mi355_device_bytes views[9] = {b->intermediates, b->weights, b->routes, b->codes, b->deltas, b->sums, b->rawdots, b->status, b->aggregate_status};
    for (size_t i = 0; i < 9; ++i) {
        if (i == 8 && views[i].address == 0 && views[i].bytes == 0) continue;
        STRIX_REQUIRE(!a8_overlap(plan, views[i]), "A8 down union views and the plan must be disjoint");
    }
    return MI355_OK;
}

// the bundle of the single-row entry points: no plan, no job word of its own, R contiguous single-row extents per view
inline RowsK a8_rows(const mi355_moe_weights& w) {
    return rows_k(mi355_moe_rows{}, w);
}

}  // namespace strix950

using namespace strix950;

extern "C" {

int32_t mi355_a8_validate(const mi355_a8_request* q, const mi355_a8_bindings* b) { return a8_validate(q, b); }
int32_t mi355_a8_validate_down(const mi355_a8_down_request* q, const mi355_a8_down_bindings* b, uint32_t logical_rows) {
    return a8_validate_down(q, b, logical_rows);
}

namespace {
// Probe of R logical rows. union_plan == nullptr: item i = assignment i (an expert chosen by two rows is read twice);
// otherwise the plan is built first and the items are its entries (each distinct expert read once).
enum { kA8PrologueProbe = 0, kA8PrologueSerial = 1, kA8PrologueQuantize = 2, kA8PrologueQuantizeOnly = 3 };
int32_t a8_probe(const mi355_a8_request* q, const mi355_a8_bindings* b, uint32_t* union_plan, hipStream_t st, int prologue_form = kA8PrologueProbe,
                 float* clear = nullptr, uint32_t clear_words = 0, const float* route_weights = nullptr) {
    const mi355_a8_shape& s = q->shape;
    const uint32_t R = s.logical_rows, groups = s.hidden / 32U;
    const uint8_t* x = reinterpret_cast<const uint8_t*>(b->input.address);
    const uint32_t* routes = reinterpret_cast<const uint32_t*>(b->routes.address);
    uint32_t* status = reinterpret_cast<uint32_t*>(b->status.address);
    if (prologue_form == kA8PrologueProbe) {
        const dim3 pgrid((groups + 7U) / 8U + (union_plan ? 1U : 0U), R);
        const uint32_t checked = union_plan ? 0U : s.top_k;       // (the union builder has checked the routes)
        const auto prologue = [&](auto kind) {
            a8_probe_prologue_kernel<decltype(kind)::value><<<pgrid, 256, 0, st>>>(x, s.hidden, routes, s.experts, checked,
                reinterpret_cast<int8_t*>(b->codes.address), reinterpret_cast<float*>(b->deltas.address), reinterpret_cast<int32_t*>(b->sums.address), status,
                union_plan, s.top_k);
        };
        if (q->input == MI355_INPUT_F32) prologue(std::integral_constant<int, 0>{});
        else if (q->input == MI355_INPUT_F16) prologue(std::integral_constant<int, 1>{});
        else prologue(std::integral_constant<int, 2>{});
    } else {
        const auto prologue = [&](auto kind, auto serial) {
            a8_serial_prologue_kernel<decltype(kind)::value, decltype(serial)::value><<<1, 1024, 0, st>>>(x, routes, route_weights, clear, clear_words,
                s.hidden, s.top_k, s.experts, reinterpret_cast<int8_t*>(b->codes.address), reinterpret_cast<float*>(b->deltas.address),
                reinterpret_cast<int32_t*>(b->sums.address), status);
        };
        const auto by_kind = [&](auto serial) {
            if (q->input == MI355_INPUT_F32) prologue(std::integral_constant<int, 0>{}, serial);
            else if (q->input == MI355_INPUT_F16) prologue(std::integral_constant<int, 1>{}, serial);
            else prologue(std::integral_constant<int, 2>{}, serial);
        };
        if (prologue_form == kA8PrologueSerial) by_kind(std::true_type{}); else by_kind(std::false_type{});
        if (prologue_form == kA8PrologueQuantizeOnly) return MI355_OK;
    }
    mi355_moe_weights w{};
    w.hidden = s.hidden; w.ffn = s.rows; w.experts = s.experts; w.top_k = s.top_k; w.gate_type = q->gate_type; w.down_type = MI355_TYPE_Q4_K;
    w.gate = reinterpret_cast<const uint8_t*>(b->gate.address); w.up = reinterpret_cast<const uint8_t*>(b->up.address);
    w.gate_row_stride = moe_row_bytes(q->gate_type, s.hidden); w.gate_expert_stride = w.gate_row_stride * s.rows;
    w.exp_kind = MI355_EXP_GFX1151; w.swiglu_limit = INFINITY;
    // projection only: output[(assignment * 2 + which) * rows + row], no image of h
    RowsK r = a8_rows(w);
    r.routes = routes;
    r.in = dense_image(reinterpret_cast<int8_t*>(b->codes.address), reinterpret_cast<float*>(b->deltas.address), reinterpret_cast<int32_t*>(b->sums.address), s.hidden);
    r.status = status; r.job_status = status;
    r.status_rs = 0;                // one shared status word
    r.clean_only = 1U;              // a step flagged by the prologue leaves `output` as it was
    r.gate_out = reinterpret_cast<float*>(b->output.address); r.up_out = r.gate_out + s.rows; r.slot_stride = 2ULL * s.rows;
    r.inter_rs = 4ULL * s.top_k * r.slot_stride;
    r.union_plan = union_plan;
    const uint32_t items = R * s.top_k;
    // the holders of an entry share the sweeps of its expert's rows, four to a sweep (a fifth holder starts a second pass, which
    // the cache serves: 8 rows x top-16 over 64 experts take 51.2 us this way against 55.6 us with eight-row sweeps)
    if (union_plan) launch_project_nb<4>(w, r, R, dim3(s.rows / 32U, items), st);
    else if (q->gate_type == MI355_TYPE_Q5_K) project_q5k_kernel<4><<<dim3(s.rows / 32U, items), 256, 0, st>>>(w, r, items);
    else if (items <= 16U) project_quad_kernel<4><<<dim3(s.rows / 32U, items), 256, 0, st>>>(w, r, items);
    else if (items <= kQuadMaxItems) project_quad_kernel<2><<<dim3(s.rows / 32U, items), 256, 0, st>>>(w, r, items);
    else launch_project_nb<4>(w, r, R, dim3(s.rows / 32U, items), st);
    return MI355_OK;
}
}  // namespace

int32_t mi355_a8_enqueue_probe(const mi355_a8_request* q, const mi355_a8_bindings* b, mi355_stream stream) {
    if (const int32_t rc = a8_validate(q, b)) return rc;          // the whole bundle is validated before the first enqueue
    // one logical row is the reference's own form (src/hip_moe_q4k_a8_probe.hip:487-502): its one-workgroup quantiser, which leaves
    // the previous image in place when the step is flagged; several rows share the status word and take the many-workgroup prologue
    a8_probe(q, b, nullptr, hs(stream), q->shape.logical_rows == 1U ? kA8PrologueQuantize : kA8PrologueProbe);
    STRIX_LAUNCHED("A8 probe");
    return MI355_OK;
}

// The serial row's step with its glue folded into the prologue (enqueue_serial_prologue_probe, include/strix/hip_moe_q4k_a8_probe.hpp:20-23,
// src/hip_moe_q4k_a8_probe.hip:503-519): clear + route and route-weight check + quantiser in one workgroup, status overwritten, then the
// projection. One logical row.
int32_t mi355_a8_enqueue_serial_prologue_probe(const mi355_a8_request* q, const mi355_a8_bindings* b, float* clear, uint32_t clear_words,
                                               const float* route_weights, mi355_stream stream) {
    if (const int32_t rc = a8_validate(q, b)) return rc;
    STRIX_REQUIRE(clear && route_weights && aligned(clear, 4) && aligned(route_weights, 4), "A8 serial prologue bindings are invalid");   // :507
    STRIX_REQUIRE(q->shape.logical_rows == 1U, "A8 serial prologue: one logical row");
    a8_probe(q, b, nullptr, hs(stream), kA8PrologueSerial, clear, clear_words, route_weights);
    STRIX_LAUNCHED("A8 serial prologue probe");
    return MI355_OK;
}

// Route check + quantiser without the projection (enqueue_quantize_only, include/strix/hip_moe_q4k_a8_probe.hpp:24,
// src/hip_moe_q4k_a8_probe.hip:540-554): status is ORed into, and a row whose status is already set is not quantised. One logical row.
int32_t mi355_a8_enqueue_quantize_only(const mi355_a8_request* q, const mi355_a8_bindings* b, mi355_stream stream) {
    if (const int32_t rc = a8_validate(q, b)) return rc;
    STRIX_REQUIRE(q->shape.logical_rows == 1U, "A8 quantize only: one logical row");
    a8_probe(q, b, nullptr, hs(stream), kA8PrologueQuantizeOnly);
    STRIX_LAUNCHED("A8 quantize only");
    return MI355_OK;
}

int32_t mi355_a8_validate_union(const mi355_a8_request* q, const mi355_a8_bindings* b, mi355_device_bytes plan) { return a8_validate_union(q, b, plan); }
int32_t mi355_a8_validate_down_union(const mi355_a8_down_request* q, const mi355_a8_down_bindings* b, uint32_t rows, mi355_device_bytes plan) {
    return a8_validate_down_union(q, b, rows, plan);
}

int32_t mi355_a8_enqueue_probe_union(const mi355_a8_request* q, const mi355_a8_bindings* b, mi355_device_bytes plan, mi355_stream stream) {
    if (const int32_t rc = a8_validate_union(q, b, plan)) return rc;
    a8_probe(q, b, reinterpret_cast<uint32_t*>(plan.address), hs(stream));
    STRIX_LAUNCHED("A8 union probe");
    return MI355_OK;
}

int32_t mi355_a8_enqueue_down_activation_quantize(const mi355_a8_down_request* q, const mi355_a8_down_bindings* b, uint32_t logical_rows,
                                                  uint32_t exp_kind, mi355_stream stream) {
    if (const int32_t rc = a8_validate_down(q, b, logical_rows)) return rc;
    STRIX_REQUIRE(exp_kind <= MI355_EXP_DECLARED, "A8 down: unknown exp kind");
    const mi355_a8_down_shape& s = q->shape;
    const uint32_t items = logical_rows * s.top_k;
    a8_down_activation_kernel<<<dim3((s.intermediate / 32U + 7U) / 8U, items), 256, 0, hs(stream)>>>(
        reinterpret_cast<float*>(b->intermediates.address), reinterpret_cast<const uint32_t*>(b->routes.address), s.experts, s.intermediate, exp_kind, q->swiglu_limit,
        reinterpret_cast<int8_t*>(b->codes.address), reinterpret_cast<float*>(b->deltas.address), reinterpret_cast<int32_t*>(b->sums.address),
        reinterpret_cast<uint32_t*>(b->status.address), reinterpret_cast<uint32_t*>(b->aggregate_status.address));
    STRIX_LAUNCHED("A8 down activation");
    return MI355_OK;
}

namespace {
int32_t a8_down_rawdots(const mi355_a8_down_request* q, const mi355_a8_down_bindings* b, uint32_t logical_rows, hipStream_t st,
                        const uint32_t* union_plan = nullptr) {
    const mi355_a8_down_shape& s = q->shape;
    mi355_moe_weights w{};
    w.hidden = s.hidden; w.ffn = s.intermediate; w.experts = s.experts; w.top_k = s.top_k; w.gate_type = MI355_TYPE_Q4_K; w.down_type = q->weight_type;
    w.down = reinterpret_cast<const uint8_t*>(b->weights.address);
    w.down_row_stride = a8_down_row_bytes(q->weight_type, s.intermediate); w.down_expert_stride = w.down_row_stride * s.hidden;
    w.swiglu_limit = INFINITY;
    RowsK r = a8_rows(w);
    r.routes = reinterpret_cast<const uint32_t*>(b->routes.address);
    r.h = dense_image(reinterpret_cast<int8_t*>(b->codes.address), reinterpret_cast<float*>(b->deltas.address), reinterpret_cast<int32_t*>(b->sums.address), s.intermediate);
    r.rawdots = reinterpret_cast<float*>(b->rawdots.address);
    r.status = reinterpret_cast<uint32_t*>(b->status.address);
    r.status_rs = 0;
    r.job_status = r.status;        // a non-finite projection recorded by the producer (bit 8) skips the rows, as in the layer entries
    r.aggregate = reinterpret_cast<uint32_t*>(b->aggregate_status.address);      // (optional: 0 = not bound)
    const uint32_t items = logical_rows * s.top_k;
    r.union_plan = union_plan;
    if (union_plan) {               // K-quant only: the items are the plan's entries
        if (q->weight_type == MI355_TYPE_Q6_K) launch_down_q6k(w, r, dim3(s.hidden / kDownGroupsRows, items), items, 0U, 0U, st);
        else if (logical_rows > 4U) launch_down_nb<8>(w, r, logical_rows, dim3(s.hidden / 64U, items), st);
        else launch_down_nb<4>(w, r, logical_rows, dim3(s.hidden / 64U, items), st);
    } else if (q->weight_type != MI355_TYPE_Q4_K) {
        const dim3 grid(s.hidden / kDownGroupsRows, items);
        if (q->weight_type == MI355_TYPE_Q8_0) down_groups_kernel<0><<<grid, 256, 0, st>>>(w, r, items, 0U, 0U);
        else if (q->weight_type == MI355_TYPE_Q5_1) down_groups_kernel<1><<<grid, 256, 0, st>>>(w, r, items, 0U, 0U);
        else launch_down_q6k(w, r, grid, items, 0U, 0U, st);
    } else if (items <= 16U) down_quad_kernel<4><<<dim3(s.hidden / 64U, items), 256, 0, st>>>(w, r, items);
    else if (items <= kQuadMaxItems) down_quad_kernel<2><<<dim3(s.hidden / 64U, items), 256, 0, st>>>(w, r, items);
    else launch_down_nb<4>(w, r, logical_rows, dim3(s.hidden / 64U, items), st);
    return MI355_OK;
}
}  // namespace

int32_t mi355_a8_enqueue_down_rawdots(const mi355_a8_down_request* q, const mi355_a8_down_bindings* b, uint32_t logical_rows, mi355_stream stream) {
    if (const int32_t rc = a8_validate_down(q, b, logical_rows)) return rc;
    a8_down_rawdots(q, b, logical_rows, hs(stream));
    STRIX_LAUNCHED("A8 down rawdots");
    return MI355_OK;
}

int32_t mi355_a8_enqueue_down_activation_quantize_union(const mi355_a8_down_request* q, const mi355_a8_down_bindings* b, uint32_t rows,
                                                        mi355_device_bytes plan, uint32_t exp_kind, mi355_stream stream) {
    if (const int32_t rc = a8_validate_down_union(q, b, rows, plan)) return rc;
    // elementwise per (row, slot): the plan is admitted with the bundle and not read
    return mi355_a8_enqueue_down_activation_quantize(q, b, rows, exp_kind, stream);
}

int32_t mi355_a8_enqueue_down_rawdots_union(const mi355_a8_down_request* q, const mi355_a8_down_bindings* b, uint32_t rows, mi355_device_bytes plan,
                                            mi355_stream stream) {
    if (const int32_t rc = a8_validate_down_union(q, b, rows, plan)) return rc;
    a8_down_rawdots(q, b, rows, hs(stream), reinterpret_cast<const uint32_t*>(plan.address));
    STRIX_LAUNCHED("A8 union down rawdots");
    return MI355_OK;
}

int32_t mi355_a8_enqueue_down_rawdots_merge(const mi355_a8_down_request* q, const mi355_a8_down_bindings* b, const mi355_slot_merge_tail* tail,
                                            mi355_stream stream) {
    if (const int32_t rc = a8_validate_down(q, b, 1)) return rc;
    STRIX_REQUIRE(tail && tail->route_weights && tail->accumulation && tail->output && tail->record && q->shape.hidden % 64U == 0 && q->shape.top_k <= 16U,
                  "A8 down slot-merge tail requires weights, accumulation, output, record, H % 64 == 0, K <= 16");
    a8_down_rawdots(q, b, 1, hs(stream));
    SlotMergeArgs t{};
    t.rawdots = reinterpret_cast<const float*>(b->rawdots.address); t.routes = reinterpret_cast<const uint32_t*>(b->routes.address);
    t.status = reinterpret_cast<uint32_t*>(b->status.address); t.hidden = q->shape.hidden; t.experts = q->shape.experts; t.top_k = q->shape.top_k;
    t.route_weights = tail->route_weights; t.accumulation = tail->accumulation; t.output = tail->output; t.output_bf16 = tail->output_bf16;
    t.bf16_commit = tail->bf16_commit; t.record = static_cast<uint32_t*>(tail->record); t.domain = tail->domain;
    a8_slot_merge_kernel<<<1, 1024, 0, hs(stream)>>>(t);
    STRIX_LAUNCHED("A8 down rawdots + slot merge");
    return MI355_OK;
}

}  // extern "C"
