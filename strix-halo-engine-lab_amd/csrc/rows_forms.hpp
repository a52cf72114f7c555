// Two more shapes of the per-row views, on the same expert kernels:
//   * the strided form: every view is {base, stride in bytes}, row r at base + r * stride, as the reference's multi-row entry
//     binds it (Rows / Strided<T>, include/strix/cuda/qwen_moe.hpp:34-37,55-76; the stages are its enqueue_prologue .. enqueue_commit,
//     :96-110, src/cuda/models/qwen/qwen_moe.cu:60-106,287-340 = the HIP known-rows launcher's kernels);
//   * the job form of the host executor (Job / Assignment / RowA8, src/cpu/core/routed_expert.hpp:41-61; Executor::run,
//     src/cpu/core/routed_expert.cpp:403-447): a list of (row, slot, expert) assignments over per-row A8 images.
#pragma once

namespace strix950 {

// ------------------------------------------------------------------------------------------------------ strided form
template <class T> __device__ __forceinline__ T* row_at(const mi355_strided& v, uint32_t row) {
    return reinterpret_cast<T*>(static_cast<uint8_t*>(v.base) + row * v.stride);
}

// One workgroup per row (src/cuda/models/qwen/qwen_moe.cu:60-106): zero the first clear_words floats of the row's accumulation,
// check the routes (an expert id out of range or a non-finite route weight: status = 1, the row is not quantised), quantise
// the input (non-finite value: bit 2, taken as 0; a delta that underflows to 0: bit 4, taken as 1; no tiny-group rule: the
// "noflush" quantiser of the probe contract, src/moe_q4k_a8_contract.cpp:67-91), store the image only for a clean row, and
// OVERWRITE the row's status word.
template <int KIND>
__global__ __launch_bounds__(256) void strided_prologue_kernel(mi355_moe_rows_strided v, uint32_t hidden, uint32_t experts, uint32_t top_k,
                                                               uint32_t clear_words) {
    extern __shared__ __attribute__((aligned(16))) uint8_t staged[];          // codes [hidden] | deltas [hidden / 32] | sums [hidden / 32]
    __shared__ uint32_t route_bits, bad;
    const uint32_t row = blockIdx.x, t = threadIdx.x, lane = t & 31U, group0 = t >> 5, groups = hidden / 32U;
    int8_t* local_codes = reinterpret_cast<int8_t*>(staged);
    float* local_deltas = reinterpret_cast<float*>(staged + hidden);
    int32_t* local_sums = reinterpret_cast<int32_t*>(staged + hidden + 4U * groups);
    if (t == 0) { route_bits = 0; bad = 0; }
    float* clear = row_at<float>(v.accumulation, row);
    for (uint32_t i = t; i < clear_words; i += 256U) clear[i] = 0.0F;
    __syncthreads();
    if (t < top_k && (row_at<const uint32_t>(v.routes, row)[t] >= experts || !finite_f(row_at<const float>(v.route_weights, row)[t])))
        atomicOr(&route_bits, static_cast<uint32_t>(MI355_STATUS_INVALID_ROUTE));
    __syncthreads();
    if (route_bits == 0U) {
        const void* input = row_at<const uint8_t>(v.input, row);
        for (uint32_t g = group0; g < groups; g += 8U) {
            float x = load_activation<KIND>(input, g * 32U + lane);
            if (!finite_f(x)) { atomicOr(&bad, static_cast<uint32_t>(MI355_STATUS_NONFINITE_ACTIVATION)); x = 0.0F; }
            const float amax = max32(__builtin_fabsf(x));
            float delta = amax == 0.0F ? 1.0F : amax / 127.0F;
            if (!(delta > 0.0F) || !finite_f(delta)) { atomicOr(&bad, static_cast<uint32_t>(MI355_STATUS_INVALID_DELTA)); delta = 1.0F; }
            const int code = a8_code(x, delta, false);
            const int sum = sum32_i(code);
            local_codes[g * 32U + lane] = static_cast<int8_t>(code);
            if (lane == 0) { local_deltas[g] = delta; local_sums[g] = sum; }
        }
    }
    __syncthreads();
    const uint32_t failure = route_bits | bad;
    if (failure == 0U) {
        uint4* codes = row_at<uint4>(v.codes, row);
        for (uint32_t i = t; i < hidden / 16U; i += 256U) codes[i] = reinterpret_cast<const uint4*>(local_codes)[i];
        for (uint32_t i = t; i < groups; i += 256U) {
            row_at<float>(v.deltas, row)[i] = local_deltas[i];
            row_at<int32_t>(v.sums, row)[i] = local_sums[i];
        }
    }
    if (t == 0) *row_at<uint32_t>(v.status, row) = failure;
}

// The job word after the plan: the OR of every row's status (the reference's CSR summary word 0, which fails the whole step).
__global__ __launch_bounds__(1024) void strided_job_status_kernel(mi355_strided status, uint32_t rows, uint32_t* job_status) {
    __shared__ uint32_t any;
    if (threadIdx.x == 0) any = 0;
    __syncthreads();
    uint32_t mine = 0;
    for (uint32_t r = threadIdx.x; r < rows; r += 1024U) mine |= *row_at<const uint32_t>(status, r);
    if (mine) atomicOr(&any, mine);
    __syncthreads();
    if (threadIdx.x == 0) *job_status = any;
}

// merge (src/cuda/models/qwen/qwen_moe.cu:287-310): nothing for a failed job or row; accumulation[o] = the fma chain over the slots
// from +0 in slot order (a NaN canonical); a value at or beyond the commit threshold flags the row and the job (bit 8).
__global__ __launch_bounds__(256) void strided_merge_kernel(mi355_moe_rows_strided v, uint32_t hidden, uint32_t experts, uint32_t top_k) {
    const uint32_t row = blockIdx.y, o = blockIdx.x * 256U + threadIdx.x;
    uint32_t* status = row_at<uint32_t>(v.status, row);
    if (*v.job_status || *status) return;
    if (o >= hidden) return;
    const uint32_t* routes = row_at<const uint32_t>(v.routes, row);
    for (uint32_t k = 0; k < top_k; ++k)
        if (routes[k] >= experts) return;
    const float* rawdots = row_at<const float>(v.rawdots, row);
    const float* weights = row_at<const float>(v.route_weights, row);
    float current = 0.0F;
    for (uint32_t k = 0; k < top_k; ++k) current = __builtin_fmaf(weights[k], rawdots[static_cast<size_t>(k) * hidden + o], current);
    row_at<float>(v.accumulation, row)[o] = current != current ? f_of(0x7fc00000U) : current;
    if ((b_of(current) & 0x7fffffffU) >= (v.output_kind == MI355_INPUT_BF16 ? 0x7f7f8000U : 0x7f800000U)) {
        atomicOr(status, 8U);
        atomicOr(v.job_status, 8U);
    }
}

// commit (src/cuda/models/qwen/qwen_moe.cu:312-340): block (0, 0) records the first failed row as DeferredMoeFirstError
// {domain, bits} (the first record of the stream stays); a failed job commits no row; otherwise output = accumulation
// (bf16: round to nearest even).
__global__ __launch_bounds__(256) void strided_commit_kernel(mi355_moe_rows_strided v, uint32_t hidden, uint32_t rows, uint32_t* record, uint32_t domain) {
    const uint32_t failure = *v.job_status;
    if (blockIdx.x == 0 && blockIdx.y == 0) {
        __shared__ uint32_t first_bad;
        if (threadIdx.x == 0) first_bad = rows;
        __syncthreads();
        for (uint32_t r = threadIdx.x; r < rows; r += 256U)
            if (*row_at<const uint32_t>(v.status, r)) { atomicMin(&first_bad, r); break; }
        __syncthreads();
        if (threadIdx.x == 0 && first_bad < rows && record) {
            const uint32_t bits = *row_at<const uint32_t>(v.status, first_bad);
            if (bits != 0U && record[0] == 0U) { record[1] = bits; record[0] = domain; }
        }
    }
    if (failure) return;
    const uint32_t o = blockIdx.x * 256U + threadIdx.x, row = blockIdx.y;
    if (o >= hidden) return;
    const uint32_t bits = b_of(row_at<const float>(v.accumulation, row)[o]);
    if (v.output_kind == MI355_INPUT_BF16) row_at<unsigned short>(v.output, row)[o] = static_cast<unsigned short>((bits + 0x7fffU + ((bits >> 16) & 1U)) >> 16);
    else row_at<float>(v.output, row)[o] = f_of(bits);
}

inline bool strided_ok(const mi355_strided& v, size_t unit) {
    return v.base != nullptr && aligned(v.base, unit) && v.stride % unit == 0;
}

// admission of the strided bundle + the kernels' view of it
int32_t check_strided(const mi355_moe_weights* w, const mi355_moe_rows_strided* v, uint32_t rows, mi355_moe_weights& wv, RowsK& k, bool need_tensors = true) {
    STRIX_REQUIRE(w && v, "moe strided: null weights or rows");
    mi355_moe_rows shell{};                     // check_moe looks at the dense bundle's pointers: stand-ins that pass its null / alignment tests
    shell.routes = static_cast<const uint32_t*>(v->routes.base); shell.route_weights = static_cast<const float*>(v->route_weights.base);
    shell.codes = static_cast<int8_t*>(v->codes.base); shell.deltas = static_cast<float*>(v->deltas.base); shell.sums = static_cast<int32_t*>(v->sums.base);
    shell.status = static_cast<uint32_t*>(v->status.base); shell.down_codes = static_cast<int8_t*>(v->down_codes.base);
    shell.down_deltas = static_cast<float*>(v->down_deltas.base); shell.down_sums = static_cast<int32_t*>(v->down_sums.base);
    shell.rawdots = static_cast<float*>(v->rawdots.base); shell.output = static_cast<float*>(v->output.base); shell.output_stride = w->hidden;
    shell.plan = v->plan; shell.job_status = v->job_status;
    if (const int32_t rc = check_moe(w, &shell, rows, wv, kIntegerClass, need_tensors)) return rc;
    STRIX_REQUIRE(v->input_kind <= MI355_INPUT_BF16 && (v->output_kind == MI355_INPUT_BF16 || v->output_kind == MI355_INPUT_F32),
                  "moe strided: input kind must be fp32 / fp16 / bf16, output kind bf16 or fp32");
    // every base and stride is 16-byte aligned (include/strix/cuda/qwen_moe.hpp:34); routes, route weights and status are words
    STRIX_REQUIRE(strided_ok(v->input, 16) && strided_ok(v->codes, 16) && strided_ok(v->deltas, 16) && strided_ok(v->sums, 16) &&
                  strided_ok(v->accumulation, 16) && strided_ok(v->down_codes, 16) && strided_ok(v->down_deltas, 16) && strided_ok(v->down_sums, 16) &&
                  strided_ok(v->rawdots, 16) && strided_ok(v->output, 16) && strided_ok(v->routes, 4) && strided_ok(v->route_weights, 4) &&
                  strided_ok(v->status, 4) && (v->intermediates.base == nullptr || strided_ok(v->intermediates, 16)),
                  "moe strided: every view needs a 16-byte aligned base and stride (routes, route weights, status: 4)");
    const uint64_t K = wv.top_k;
    STRIX_REQUIRE(v->input.stride >= static_cast<uint64_t>(wv.hidden) * (v->input_kind == MI355_INPUT_F32 ? 4U : 2U) && v->routes.stride >= 4U * K &&
                  v->route_weights.stride >= 4U * K && v->codes.stride >= wv.hidden && v->deltas.stride >= wv.hidden / 8U && v->sums.stride >= wv.hidden / 8U &&
                  v->status.stride >= 4U && v->accumulation.stride >= 4ULL * wv.hidden && v->down_codes.stride >= K * wv.ffn &&
                  v->down_deltas.stride >= K * (wv.ffn / 8U) && v->down_sums.stride >= K * (wv.ffn / 8U) && v->rawdots.stride >= 4U * K * wv.hidden &&
                  v->output.stride >= static_cast<uint64_t>(wv.hidden) * (v->output_kind == MI355_INPUT_F32 ? 4U : 2U) &&
                  (v->intermediates.base == nullptr || v->intermediates.stride >= 8U * K * wv.ffn),
                  "moe strided: a view's stride is shorter than one row's extent");
    k = rows_k(shell, wv);
    k.in = A8Image{shell.codes, shell.deltas, shell.sums, wv.hidden, 1U, v->codes.stride, v->deltas.stride, v->sums.stride, nullptr};
    k.h = A8Image{shell.down_codes, shell.down_deltas, shell.down_sums, wv.ffn, wv.top_k, v->down_codes.stride, v->down_deltas.stride, v->down_sums.stride, nullptr};
    k.routes_rs = v->routes.stride; k.route_weights_rs = v->route_weights.stride; k.status_rs = v->status.stride;
    k.rawdots_rs = v->rawdots.stride;
    // intermediates: per slot [h (in the place of gate) | up], include/strix/cuda/qwen_moe.hpp:63
    float* inter = static_cast<float*>(v->intermediates.base);
    k.gate_out = nullptr; k.h_out = inter; k.up_out = inter ? inter + wv.ffn : nullptr;
    k.slot_stride = 2ULL * wv.ffn; k.inter_rs = v->intermediates.stride;
    k.base = nullptr; k.output = nullptr;
    return MI355_OK;
}

// The prologue of the fp16 prefill over strided rows (enqueue_prefill_prologue, include/strix/hip_moe_q4k_a8_known_rows.hpp:86-87,
// without the A8 quantiser, which the fp16 form does not use): zero the row's `clear` words, check its routes and route weights,
// OVERWRITE its status word; row 0 clears the job word.
__global__ __launch_bounds__(256) void prefill_rows_prologue_kernel(mi355_prefill_rows v, uint32_t experts, uint32_t top_k, uint32_t clear_words) {
    __shared__ uint32_t route_bits;
    const uint32_t row = blockIdx.x, t = threadIdx.x;
    if (t == 0) route_bits = 0;
    if (v.clear.base) {
        float* clear = row_at<float>(v.clear, row);
        for (uint32_t i = t; i < clear_words; i += 256U) clear[i] = 0.0F;
    }
    __syncthreads();
    const uint32_t* routes = row_at<const uint32_t>(v.routes, row);
    const float* weights = row_at<const float>(v.route_weights, row);
    for (uint32_t k = t; k < top_k; k += 256U)
        if (routes[k] >= experts || !finite_f(weights[k])) atomicOr(&route_bits, static_cast<uint32_t>(MI355_STATUS_INVALID_ROUTE));
    __syncthreads();
    if (t == 0) {
        *row_at<uint32_t>(v.status, row) = route_bits;
        if (row == 0) *v.job_status = 0U;
    }
}

// --------------------------------------------------------------------------------------------------------- job form
// The executor object of the job form: the A8 image of h for up to max_assignments assignments and the job word, allocated
// once (as Executor owns its scratch vectors, src/cpu/core/routed_expert.cpp:356-363).
struct JobExecutor {
    uint32_t max_assignments, max_ffn, exp_kind;
    int device;
    int8_t* h_codes;
    float* h_deltas;
    int32_t* h_sums;
    uint32_t* job_status;
};

__global__ void clear_word_kernel(uint32_t* word) { *word = 0U; }

}  // namespace strix950

using namespace strix950;

extern "C" {

// Known-prompt prefill over strided rows in the FAST class (known_rows::enqueue_prefill with the fp16 form,
// include/strix/hip_moe_q4k_a8_known_rows.hpp:75-111): prologue, expert plan, gate / up + SwiGLU, down rows into rawdots; the caller
// merges and commits.
int32_t mi355_moe_enqueue_prefill_rows_f16(const mi355_moe_weights* w, const mi355_prefill_rows* v, uint32_t rows, uint32_t clear_words, mi355_stream stream) {
    STRIX_REQUIRE(w && v, "moe prefill rows: null weights or rows");
    mi355_moe_rows shell{};                     // check_moe looks at the dense bundle's pointers: stand-ins that pass its null / alignment tests
    shell.routes = static_cast<const uint32_t*>(v->routes.base); shell.route_weights = static_cast<const float*>(v->route_weights.base);
    shell.status = static_cast<uint32_t*>(v->status.base); shell.rawdots = static_cast<float*>(v->rawdots.base);
    shell.plan = v->plan; shell.job_status = v->job_status; shell.h_f16 = v->h_f16;
    shell.output = static_cast<float*>(v->rawdots.base); shell.output_stride = w->hidden;
    shell.codes = reinterpret_cast<int8_t*>(v->h_f16); shell.deltas = reinterpret_cast<float*>(v->h_f16); shell.sums = reinterpret_cast<int32_t*>(v->h_f16);
    shell.down_codes = shell.codes; shell.down_deltas = shell.deltas; shell.down_sums = shell.sums;     // (the fp16 form has no A8 images)
    mi355_moe_weights wv;
    if (const int32_t rc = check_moe(w, &shell, rows, wv, kPrefillClass)) return rc;
    STRIX_REQUIRE(rows <= 65535U, "moe prefill rows: at most 65535 rows per call");
    STRIX_REQUIRE(wv.hidden % 128U == 0 && wv.ffn % 64U == 0, "moe prefill rows: hidden must be a multiple of 128, ffn of 64");
    STRIX_REQUIRE(v->h_f16 && aligned(v->h_f16, 16), "moe prefill rows: h_f16 workspace is null or misaligned");
    STRIX_REQUIRE(strided_ok(v->input, 16) && strided_ok(v->rawdots, 16) && strided_ok(v->routes, 4) && strided_ok(v->route_weights, 4) &&
                  strided_ok(v->status, 4) && (v->clear.base == nullptr || strided_ok(v->clear, 4)),
                  "moe prefill rows: input and rawdots need a 16-byte aligned base and stride (routes, route weights, status, clear: 4)");
    const uint64_t K = wv.top_k;
    STRIX_REQUIRE(v->input.stride >= 2ULL * wv.hidden && v->routes.stride >= 4U * K && v->route_weights.stride >= 4U * K && v->status.stride >= 4U &&
                  v->rawdots.stride >= 4U * K * wv.hidden, "moe prefill rows: a view's stride is shorter than one row's extent");
    STRIX_REQUIRE(clear_words == 0 || (v->clear.base && (rows == 1U || 4ULL * clear_words <= v->clear.stride)),
                  "moe prefill rows: clear_words needs the clear view and must stay inside a row's stride");
    hipStream_t st = hs(stream);
    prefill_rows_prologue_kernel<<<rows, 256, 0, st>>>(*v, wv.experts, wv.top_k, clear_words);
    const PrefillViews views{v->input.base, v->input.stride, RoutesView{shell.routes, v->routes.stride, wv.top_k}, shell.status, v->status.stride,
                             v->job_status, shell.rawdots, v->rawdots.stride, v->rawdots_bf16 ? 1U : 0U, v->plan, v->h_f16};
    return enqueue_prefill_core(wv, views, rows, st);
}

int32_t mi355_moe_strided_enqueue_prologue(const mi355_moe_weights* w, const mi355_moe_rows_strided* v, uint32_t rows, uint32_t clear_words, mi355_stream stream) {
    mi355_moe_weights wv; RowsK k;
    if (const int32_t rc = check_strided(w, v, rows, wv, k, false)) return rc;
    STRIX_REQUIRE(clear_words * 4ULL <= v->accumulation.stride || rows == 1U, "moe strided prologue: clear_words reaches into the next row's accumulation");
    STRIX_REQUIRE(wv.hidden <= 16384U, "moe strided prologue: hidden beyond 16384");
    const size_t lds = wv.hidden + 8U * (wv.hidden / 32U);
    hipStream_t st = hs(stream);
    if (v->input_kind == MI355_INPUT_F32) strided_prologue_kernel<0><<<rows, 256, lds, st>>>(*v, wv.hidden, wv.experts, wv.top_k, clear_words);
    else if (v->input_kind == MI355_INPUT_F16) strided_prologue_kernel<1><<<rows, 256, lds, st>>>(*v, wv.hidden, wv.experts, wv.top_k, clear_words);
    else strided_prologue_kernel<2><<<rows, 256, lds, st>>>(*v, wv.hidden, wv.experts, wv.top_k, clear_words);
    STRIX_LAUNCHED("moe strided prologue");
    return MI355_OK;
}

int32_t mi355_moe_strided_enqueue_csr(const mi355_moe_weights* w, const mi355_moe_rows_strided* v, uint32_t rows, mi355_stream stream) {
    mi355_moe_weights wv; RowsK k;
    if (const int32_t rc = check_strided(w, v, rows, wv, k, false)) return rc;
    hipStream_t st = hs(stream);
    launch_plan(RoutesView{k.routes, k.routes_rs, wv.top_k}, wv.experts, rows * wv.top_k, plan_split(wv, rows), item_bound(wv, rows), v->plan, st);
    strided_job_status_kernel<<<1, 1024, 0, st>>>(v->status, rows, v->job_status);
    STRIX_LAUNCHED("moe strided plan");
    return MI355_OK;
}

int32_t mi355_moe_strided_enqueue_project(const mi355_moe_weights* w, const mi355_moe_rows_strided* v, uint32_t rows, mi355_stream stream) {
    mi355_moe_weights wv; RowsK k;
    if (const int32_t rc = check_strided(w, v, rows, wv, k)) return rc;
    launch_project(wv, k, rows, item_bound(wv, rows), hs(stream));
    STRIX_LAUNCHED("moe strided project");
    return MI355_OK;
}

int32_t mi355_moe_strided_enqueue_down(const mi355_moe_weights* w, const mi355_moe_rows_strided* v, uint32_t rows, mi355_stream stream) {
    mi355_moe_weights wv; RowsK k;
    if (const int32_t rc = check_strided(w, v, rows, wv, k)) return rc;
    launch_down(wv, k, rows, item_bound(wv, rows), hs(stream));
    STRIX_LAUNCHED("moe strided down");
    return MI355_OK;
}

int32_t mi355_moe_strided_enqueue_merge(const mi355_moe_weights* w, const mi355_moe_rows_strided* v, uint32_t rows, mi355_stream stream) {
    mi355_moe_weights wv; RowsK k;
    if (const int32_t rc = check_strided(w, v, rows, wv, k, false)) return rc;
    strided_merge_kernel<<<dim3((wv.hidden + 255U) / 256U, rows), 256, 0, hs(stream)>>>(*v, wv.hidden, wv.experts, wv.top_k);
    STRIX_LAUNCHED("moe strided merge");
    return MI355_OK;
}

int32_t mi355_moe_strided_enqueue_commit(const mi355_moe_weights* w, const mi355_moe_rows_strided* v, uint32_t rows, uint32_t* record, uint32_t domain,
                                         mi355_stream stream) {
    mi355_moe_weights wv; RowsK k;
    if (const int32_t rc = check_strided(w, v, rows, wv, k, false)) return rc;
    strided_commit_kernel<<<dim3((wv.hidden + 255U) / 256U, rows), 256, 0, hs(stream)>>>(*v, wv.hidden, rows, record, domain);
    STRIX_LAUNCHED("moe strided commit");
    return MI355_OK;
}

int32_t mi355_moe_strided_enqueue(const mi355_moe_weights* w, const mi355_moe_rows_strided* v, uint32_t rows, uint32_t clear_words, uint32_t* record,
                                  uint32_t domain, mi355_stream stream) {
    mi355_moe_weights wv; RowsK k;
    if (const int32_t rc = check_strided(w, v, rows, wv, k)) return rc;       // the whole bundle is validated before the first enqueue
    if (const int32_t rc = mi355_moe_strided_enqueue_prologue(w, v, rows, clear_words, stream)) return rc;
    if (const int32_t rc = mi355_moe_strided_enqueue_csr(w, v, rows, stream)) return rc;
    if (const int32_t rc = mi355_moe_strided_enqueue_project(w, v, rows, stream)) return rc;
    if (const int32_t rc = mi355_moe_strided_enqueue_down(w, v, rows, stream)) return rc;
    if (const int32_t rc = mi355_moe_strided_enqueue_merge(w, v, rows, stream)) return rc;
    return mi355_moe_strided_enqueue_commit(w, v, rows, record, domain, stream);
}

// ---------------------------------------------------------------------------------------------------------- job form
void* mi355_executor_create(uint32_t max_assignments, uint32_t max_ffn, uint32_t exp_kind) {
    if (max_assignments == 0 || max_assignments > 65535U || max_ffn == 0 || max_ffn % 128U != 0 || exp_kind > MI355_EXP_DECLARED) {
        fail(MI355_E_INVALID_ARGUMENT, "executor: max_assignments must be within 1..65535, max_ffn a positive multiple of 128, exp kind known");
        return nullptr;
    }
    JobExecutor* x = new JobExecutor{};
    x->max_assignments = max_assignments; x->max_ffn = max_ffn; x->exp_kind = exp_kind;
    const size_t n = static_cast<size_t>(max_assignments);
    hipError_t e = hipGetDevice(&x->device);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&x->h_codes), n * max_ffn);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&x->h_deltas), n * (max_ffn / 32U) * 4U);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&x->h_sums), n * (max_ffn / 32U) * 4U);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&x->job_status), 256);
    if (e != hipSuccess) {
        hip_fail(e, "executor: workspace allocation");
        (void)hipFree(x->h_codes); (void)hipFree(x->h_deltas); (void)hipFree(x->h_sums); (void)hipFree(x->job_status);
        delete x;
        return nullptr;
    }
    return x;
}

void mi355_executor_destroy(void* executor) {
    JobExecutor* x = static_cast<JobExecutor*>(executor);
    if (!x) return;
    (void)hipFree(x->h_codes); (void)hipFree(x->h_deltas); (void)hipFree(x->h_sums); (void)hipFree(x->job_status);
    delete x;
}

int32_t mi355_executor_run(void* executor, const mi355_expert_job* job, mi355_stream stream) {
    JobExecutor* x = static_cast<JobExecutor*>(executor);
    STRIX_REQUIRE(x && job, "executor: null executor or job");
    if (job->count == 0) return MI355_OK;                                    // Executor::run: an empty job is nothing
    const mi355_layer_weights& lw = job->weights;
    STRIX_REQUIRE(lw.gate_format <= 1U && lw.down_format <= 1U, "executor: gate format must be 0 (Q4_K) or 1 (Q5_K), down format 0 (Q5_1) or 1 (Q8_0)");
    STRIX_REQUIRE(lw.hidden >= 256U && lw.hidden % 256U == 0 && lw.ffn >= 128U && lw.ffn % 128U == 0, "executor: hidden must be a multiple of 256, ffn of 128");
    STRIX_REQUIRE(lw.ffn <= x->max_ffn && job->count <= x->max_assignments, "executor: the job is larger than the executor was created for");
    STRIX_REQUIRE(lw.gate && lw.up && lw.down && aligned(lw.gate, 16) && aligned(lw.up, 16) && aligned(lw.down, 16), "executor: weight tensors must be non-null and 16-byte aligned");
    STRIX_REQUIRE(job->rows && job->assignments && job->rawdots && job->status && aligned(job->rawdots, 16) && job->rawdot_row_stride % 4U == 0 &&
                  job->rawdot_row_stride >= lw.hidden, "executor: rows / assignments / rawdots / status invalid (rawdots 16-byte aligned, row stride a multiple of 4 floats)");
    mi355_moe_weights w{};
    w.hidden = lw.hidden; w.ffn = lw.ffn; w.experts = 0xffffffffU; w.top_k = 1;        // the job names its experts itself and is trusted, as on the host
    w.gate_type = lw.gate_format == 0 ? MI355_TYPE_Q4_K : MI355_TYPE_Q5_K; w.down_type = lw.down_format == 0 ? MI355_TYPE_Q5_1 : MI355_TYPE_Q8_0;
    w.gate = lw.gate; w.up = lw.up; w.down = lw.down;
    w.gate_row_stride = moe_row_bytes(w.gate_type, w.hidden); w.gate_expert_stride = w.gate_row_stride * w.ffn;
    w.down_row_stride = moe_row_bytes(w.down_type, w.ffn); w.down_expert_stride = w.down_row_stride * w.hidden;
    w.exp_kind = x->exp_kind; w.swiglu_limit = INFINITY;
    RowsK k = rows_k(mi355_moe_rows{}, w);
    k.assignments = job->assignments;
    k.in = A8Image{nullptr, nullptr, nullptr, w.hidden, 1U, 0, 0, 0, job->rows};
    k.h = dense_image(x->h_codes, x->h_deltas, x->h_sums, w.ffn);
    k.rawdots = job->rawdots; k.rawdots_rs = 4ULL * job->rawdot_row_stride;
    k.status = job->status; k.status_rs = 4; k.job_status = x->job_status;
    k.nonfinite_bit = 1U;                                                    // kNonfinite, src/cpu/core/routed_expert.hpp:51
    hipStream_t st = hs(stream);
    clear_word_kernel<<<1, 1, 0, st>>>(x->job_status);
    const uint32_t items = job->count;
    if (w.gate_type == MI355_TYPE_Q5_K) project_q5k_kernel<4><<<dim3(w.ffn / 32U, items), 256, 0, st>>>(w, k, items);
    else if (items <= 16U) project_quad_kernel<4><<<dim3(w.ffn / 32U, items), 256, 0, st>>>(w, k, items);
    else if (items <= kQuadMaxItems) project_quad_kernel<2><<<dim3(w.ffn / 32U, items), 256, 0, st>>>(w, k, items);
    else launch_project_nb<4>(w, k, items, dim3(w.ffn / 32U, items), st);
    const dim3 grid(w.hidden / kDownGroupsRows, items);
    if (w.down_type == MI355_TYPE_Q8_0) down_groups_kernel<0><<<grid, 256, 0, st>>>(w, k, items, 0U, 0U);
    else down_groups_kernel<1><<<grid, 256, 0, st>>>(w, k, items, 0U, 0U);
    STRIX_LAUNCHED("executor run");
    return MI355_OK;
}

}  // extern "C"
