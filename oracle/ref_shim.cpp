// TEST INFRASTRUCTURE. C-ABI view of the reference's own CPU functions, for validating the restated oracle
// (strix_oracle.c) bit for bit. This file holds no reference source: it includes the reference headers from
// the reference tree at build time (oracle/Makefile, target _ref) and is compiled together with the reference's
// own .cpp files into oracle/_ref/libstrix_ref.so. It is only built where the reference tree is present.
#include "cpu/core/backend.hpp"
#include "cpu/core/routed_expert.hpp"
#include "cpu/core/routed_expert_kernels.hpp"
#include "strix/ds41_moe.hpp"
#include "strix/ggml_dequant.hpp"
#include "strix/moe/activation_policy.hpp"
#include "strix/moe/combine.hpp"
#include "strix/moe/expert_union.hpp"
#include "strix/moe/route_policy.hpp"
#include "strix/moe_a8_down_contract.hpp"
#include "strix/moe_q4k_a8_contract.hpp"
#include "strix/q8_0_rule.hpp"

#include <cmath>
#include <cstdio>
#include <cstring>
#include <filesystem>
#include <memory>
#include <mutex>
#include <span>
#include <string>
#include <vector>

namespace {
namespace ex = strix::cpu::expert;
namespace a8 = strix::moe_q4k_a8;

thread_local std::string g_error;

struct DeclaredMath { static float exp(float x) { return strix::ds41::declared_exp(x); } };
struct LibmMath { static float exp(float x) { return std::exp(x); } };

// The reference constructor reads two table files; the probe tables themselves are not in the reference tree, so
// (like the reference's own host test when STRIX_EXP_TABLES is unset) synthetic files are written: here EMPTY ones,
// which make v_exp the correctly rounded exp2.
const ex::Gfx1151Exp& empty_table_exp() {
    static std::once_flag once;
    static std::unique_ptr<ex::Gfx1151Exp> exp;
    std::call_once(once, [] {
        const auto dir = std::filesystem::temp_directory_path() / ("strix_ref_empty_tables_" + std::to_string(::getpid()));
        std::filesystem::create_directories(dir);
        for (const char* name : {"tbl_exp_pm.bin", "hard_v_exp_f32.bin"}) {
            FILE* f = std::fopen((dir / name).c_str(), "wb");
            if (f) std::fclose(f);
        }
        exp = std::make_unique<ex::Gfx1151Exp>(dir.string());
        std::error_code ec;
        std::filesystem::remove_all(dir, ec);
    });
    return *exp;
}

a8::QuantizedRow make_row(const std::int8_t* codes, const float* deltas, const std::int32_t* sums, std::size_t n) {
    a8::QuantizedRow row;
    row.codes.assign(codes, codes + n);
    row.deltas.assign(deltas, deltas + n / 32);
    row.sums.assign(sums, sums + n / 32);
    return row;
}
void copy_row(const a8::QuantizedRow& row, std::int8_t* codes, float* deltas, std::int32_t* sums) {
    std::memcpy(codes, row.codes.data(), row.codes.size());
    std::memcpy(deltas, row.deltas.data(), row.deltas.size() * 4);
    std::memcpy(sums, row.sums.data(), row.sums.size() * 4);
}
template <class F> int guarded(F&& f) {
    try { f(); return 0; } catch (const std::exception& e) { g_error = e.what(); return -1; }
}
}  // namespace

extern "C" {

const char* ref_last_error() { return g_error.c_str(); }

float ref_half_to_float(std::uint16_t bits) { return strix::cpu::half_to_float(bits); }
float ref_contract_half_to_float(std::uint16_t bits) { return a8::half_bits_to_float(bits); }
float ref_ggml_fp16(std::uint16_t bits) { return strix::ggml_dequant::fp16(bits); }
float ref_declared_exp(float x) { return strix::ds41::declared_exp(x); }
float ref_gfx1151_expf_empty_tables(float x) { return empty_table_exp().expf(x); }

int ref_dequantize_row(std::uint32_t type, const std::uint8_t* row, std::size_t bytes, float* out, std::size_t n) {
    return guarded([&] {
        strix::ggml_dequant::dequantize_row(type, std::span<const std::byte>(reinterpret_cast<const std::byte*>(row), bytes),
                                            std::span<float>(out, n));
    });
}
void ref_q4k_decode_factors(const std::uint8_t* packed12, std::uint32_t group, std::uint32_t* scale, std::uint32_t* minimum) {
    const auto f = a8::decode_factors(std::span<const std::byte>(reinterpret_cast<const std::byte*>(packed12), 12), group);
    *scale = f.scale; *minimum = f.minimum;
}
void ref_q8_0_quantize_group(const float* v, float* d, std::int8_t* q) {
    const auto g = strix::q8_0::quantize_group(v);
    *d = g.d;
    std::memcpy(q, g.q, 32);
}

// CPU backend kernel table (scalar reference entries).
int ref_quantize_a8(const float* x, std::size_t width, std::int8_t* codes, float* deltas, std::int32_t* sums) {
    return guarded([&] { strix::cpu::reference_kernels().quantize_a8(x, width, codes, deltas, sums); });
}
int ref_rmsnorm_f32(const float* x, const float* w, unsigned n, float eps, float* y, unsigned rows) {
    return guarded([&] { strix::cpu::reference_kernels().rmsnorm_f32(x, w, n, eps, y, rows, strix::cpu::Stream{}); });
}
int ref_gemv_q8_0_a8(const strix::cpu::Q8a8View* view) {
    return guarded([&] { strix::cpu::reference_kernels().gemv_q8_0_a8(*view, strix::cpu::Stream{}); });
}

// Q4_K x A8 contract.
int ref_contract_quantize_f32(const float* x, std::size_t n, std::int8_t* codes, float* deltas, std::int32_t* sums) {
    return guarded([&] { copy_row(a8::quantize_f32(std::span<const float>(x, n)), codes, deltas, sums); });
}
int ref_quantize_down_values(const float* x, std::size_t n, std::int8_t* codes, float* deltas, std::int32_t* sums) {
    return guarded([&] { copy_row(a8::quantize_down_values(std::span<const float>(x, n)), codes, deltas, sums); });
}
int ref_q4k_evaluate_row(const std::uint8_t* w, std::size_t bytes, const std::int8_t* codes, const float* deltas,
                         const std::int32_t* sums, std::size_t n, float* out) {
    return guarded([&] {
        *out = a8::evaluate_row(std::span<const std::byte>(reinterpret_cast<const std::byte*>(w), bytes), make_row(codes, deltas, sums, n));
    });
}
int ref_evaluate_down_row(const std::uint8_t* w, std::size_t bytes, const std::int8_t* codes, const float* deltas,
                          const std::int32_t* sums, std::size_t n, std::uint32_t type, float* out) {
    return guarded([&] {
        *out = a8::evaluate_down_row(std::span<const std::byte>(reinterpret_cast<const std::byte*>(w), bytes),
                                     make_row(codes, deltas, sums, n), type);
    });
}

// Host routed-expert row kernels (no admission caps on the width).
void ref_gate_row_q4k(const std::uint8_t* wrow, std::uint32_t blocks, const std::int8_t* codes, const float* deltas,
                      const std::int32_t* sums, float* out) {
    const ex::RowA8 row{codes, deltas, sums};
    const ex::RowA8* rows[1] = {&row};
    ex::detail::scalar_kernels().gate[0](wrow, blocks, rows, 1, out);
}
void ref_gate_row_q5k(const std::uint8_t* wrow, std::uint32_t blocks, const std::int8_t* codes, const float* deltas,
                      const std::int32_t* sums, float* out) {
    const ex::RowA8 row{codes, deltas, sums};
    const ex::RowA8* rows[1] = {&row};
    ex::detail::scalar_kernels().gate[1](wrow, blocks, rows, 1, out);
}
void ref_down_row_q8_0(const std::uint8_t* wrow, std::uint32_t groups, const std::int8_t* codes, const float* deltas,
                       const std::int32_t* sums, float* out) {
    ex::detail::scalar_kernels().down[1](wrow, groups, &codes, &deltas, &sums, 1, out);
}

void ref_down_row_q5_1(const std::uint8_t* wrow, std::uint32_t groups, const std::int8_t* codes, const float* deltas,
                       const std::int32_t* sums, float* out) {
    ex::detail::scalar_kernels().down[0](wrow, groups, &codes, &deltas, &sums, 1, out);
}

// Whole routed-expert job (gate/up Q4_K, or Q5_K when bit 1 of down_q5_1 is set; down Q8_0, or Q5_1 when bit 0 of down_q5_1
// is set; the host executor has no Q4_K down),
// empty exp tables. assignments: count x {row, slot, expert}. executor_threads == 0: reference_run (scalar oracle);
// otherwise the pool.
int ref_routed_expert_run_fmt(std::uint32_t hidden, std::uint32_t ffn, const std::uint8_t* gate, const std::uint8_t* up,
                              const std::uint8_t* down, int down_q5_1, const std::int8_t* codes, const float* deltas,
                              const std::int32_t* sums, std::uint32_t rows, const std::uint32_t* assignments,
                              std::uint32_t count, float* rawdots, std::uint64_t rawdot_row_stride, std::uint32_t* status,
                              unsigned executor_threads, int allow_simd);
int ref_routed_expert_run(std::uint32_t hidden, std::uint32_t ffn, const std::uint8_t* gate, const std::uint8_t* up,
                          const std::uint8_t* down_q8_0, const std::int8_t* codes, const float* deltas,
                          const std::int32_t* sums, std::uint32_t rows, const std::uint32_t* assignments,
                          std::uint32_t count, float* rawdots, std::uint64_t rawdot_row_stride, std::uint32_t* status,
                          unsigned executor_threads, int allow_simd) {
    return ref_routed_expert_run_fmt(hidden, ffn, gate, up, down_q8_0, 0, codes, deltas, sums, rows, assignments, count, rawdots,
                                     rawdot_row_stride, status, executor_threads, allow_simd);
}
int ref_routed_expert_run_fmt(std::uint32_t hidden, std::uint32_t ffn, const std::uint8_t* gate, const std::uint8_t* up,
                              const std::uint8_t* down_q8_0, int down_q5_1, const std::int8_t* codes, const float* deltas,
                              const std::int32_t* sums, std::uint32_t rows, const std::uint32_t* assignments,
                              std::uint32_t count, float* rawdots, std::uint64_t rawdot_row_stride, std::uint32_t* status,
                              unsigned executor_threads, int allow_simd) {
    return guarded([&] {
        std::vector<ex::RowA8> row_views(rows);
        for (std::uint32_t r = 0; r < rows; ++r)
            row_views[r] = {codes + std::size_t{r} * hidden, deltas + std::size_t{r} * (hidden / 32), sums + std::size_t{r} * (hidden / 32)};
        std::vector<ex::Assignment> as(count);
        for (std::uint32_t a = 0; a < count; ++a) as[a] = {assignments[3 * a], assignments[3 * a + 1], assignments[3 * a + 2]};
        ex::Job job;
        job.weights = {gate, up, down_q8_0, (down_q5_1 & 2) ? ex::GateFormat::q5_k : ex::GateFormat::q4_k,
                       (down_q5_1 & 1) ? ex::DownFormat::q5_1 : ex::DownFormat::q8_0, {hidden, ffn}};
        job.rows = row_views.data(); job.assignments = as.data(); job.count = count;
        job.rawdots = rawdots; job.rawdot_row_stride = rawdot_row_stride; job.status = status;
        if (executor_threads == 0) ex::reference_run(job, empty_table_exp());
        else { ex::Executor pool(executor_threads, empty_table_exp(), allow_simd != 0); pool.run(job); }
    });
}

// Persistent pool for timing (cpu_baseline kind "reference" on shapes the host executor supports).
void* ref_executor_create(unsigned threads, int allow_simd) {
    try { return new ex::Executor(threads, empty_table_exp(), allow_simd != 0); } catch (const std::exception& e) { g_error = e.what(); return nullptr; }
}
const char* ref_executor_isa(void* pool) { return static_cast<ex::Executor*>(pool)->isa(); }
// One job on the persistent pool (arguments as ref_routed_expert_run_fmt).
int ref_executor_run(void* pool, std::uint32_t hidden, std::uint32_t ffn, const std::uint8_t* gate, const std::uint8_t* up,
                     const std::uint8_t* down, int down_q5_1, const std::int8_t* codes, const float* deltas, const std::int32_t* sums,
                     std::uint32_t rows, const std::uint32_t* assignments, std::uint32_t count, float* rawdots,
                     std::uint64_t rawdot_row_stride, std::uint32_t* status) {
    return guarded([&] {
        std::vector<ex::RowA8> row_views(rows);
        for (std::uint32_t r = 0; r < rows; ++r)
            row_views[r] = {codes + std::size_t{r} * hidden, deltas + std::size_t{r} * (hidden / 32), sums + std::size_t{r} * (hidden / 32)};
        std::vector<ex::Assignment> as(count);
        for (std::uint32_t a = 0; a < count; ++a) as[a] = {assignments[3 * a], assignments[3 * a + 1], assignments[3 * a + 2]};
        ex::Job job;
        job.weights = {gate, up, down, (down_q5_1 & 2) ? ex::GateFormat::q5_k : ex::GateFormat::q4_k,
                       (down_q5_1 & 1) ? ex::DownFormat::q5_1 : ex::DownFormat::q8_0, {hidden, ffn}};
        job.rows = row_views.data(); job.assignments = as.data(); job.count = count;
        job.rawdots = rawdots; job.rawdot_row_stride = rawdot_row_stride; job.status = status;
        static_cast<ex::Executor*>(pool)->run(job);
    });
}
void ref_executor_destroy(void* pool) { delete static_cast<ex::Executor*>(pool); }

// Router policy (softmax scores with a Math trait, then selection and weights).
int ref_route_scores_softmax(const float* logits, std::size_t n, float* scores, int libm_exp) {
    return guarded([&] {
        if (libm_exp) strix::moe::route_scores_ref<LibmMath>(strix::moe::RouteScore::softmax, std::span<const float>(logits, n), std::span<float>(scores, n));
        else strix::moe::route_scores_ref<DeclaredMath>(strix::moe::RouteScore::softmax, std::span<const float>(logits, n), std::span<float>(scores, n));
    });
}
int ref_route_select(std::uint32_t experts, std::uint32_t top_k, float renorm_eps, float scale, int renormalize,
                     const float* scores, std::uint32_t* ids, float* weights) {
    return guarded([&] {
        strix::moe::RoutePolicy p;
        p.score = strix::moe::RouteScore::softmax; p.selection_bias = false; p.key = strix::moe::RouteKey::float_serial;
        p.order = strix::moe::RouteOrder::selection; p.experts = experts; p.top_k = top_k;
        p.renormalize = renormalize != 0; p.renorm_single = true; p.renorm_eps = renorm_eps; p.scale = scale;
        strix::moe::route_select_ref(p, std::span<const float>(scores, experts), {}, std::span<std::uint32_t>(ids, top_k),
                                     std::span<float>(weights, top_k));
    });
}
// The same with the policy's renorm_single field given (top_k = 1 renormalises only when it is set).
int ref_route_select_policy(std::uint32_t experts, std::uint32_t top_k, float renorm_eps, float scale, int renormalize, int renorm_single,
                            const float* scores, std::uint32_t* ids, float* weights) {
    return guarded([&] {
        strix::moe::RoutePolicy p;
        p.score = strix::moe::RouteScore::softmax; p.selection_bias = false; p.key = strix::moe::RouteKey::float_serial;
        p.order = strix::moe::RouteOrder::selection; p.experts = experts; p.top_k = top_k;
        p.renormalize = renormalize != 0; p.renorm_single = renorm_single != 0; p.renorm_eps = renorm_eps; p.scale = scale;
        strix::moe::route_select_ref(p, std::span<const float>(scores, experts), {}, std::span<std::uint32_t>(ids, top_k),
                                     std::span<float>(weights, top_k));
    });
}
// The SwiGLU clamp trait.
// validate / validate_down of the two A8 contracts (src/moe_q4k_a8_contract.cpp:343-372, src/moe_a8_down_contract.cpp:53-82):
// 0 = admitted, -1 = refused (ref_last_error holds the reason). views: nine {address, bytes} pairs in the order of Bindings /
// DownBindings.
int ref_a8_validate(int enabled, const char* identity, int input_fp32, std::uint32_t hidden, std::uint32_t rows, std::uint32_t experts,
                    std::uint32_t top_k, std::uint32_t logical_rows, std::uint32_t gate_type, std::uint32_t up_type, int fused, float limit,
                    const std::uint64_t* views) {
    a8::Request q;
    q.enabled = enabled != 0; q.approved_numerical_identity = identity ? std::string_view(identity) : std::string_view();
    q.input = input_fp32 ? a8::InputKind::fp32 : a8::InputKind::bf16;
    q.shape = a8::Shape{hidden, rows, experts, top_k, logical_rows};
    q.gate_type = gate_type; q.up_type = up_type; q.fused_gate_up = fused != 0; q.swiglu_limit = limit;
    a8::DeviceBytes v[9];
    for (int i = 0; i < 9; ++i) v[i] = a8::DeviceBytes{static_cast<std::uintptr_t>(views[2 * i]), views[2 * i + 1]};
    const a8::Bindings b{v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], v[8]};
    return guarded([&] { a8::validate(q, b); });
}
int ref_a8_validate_down(int enabled, const char* identity, std::uint32_t hidden, std::uint32_t intermediate, std::uint32_t experts,
                         std::uint32_t top_k, std::uint32_t weight_type, float limit, const std::uint64_t* views) {
    a8::DownRequest q;
    q.enabled = enabled != 0; q.approved_numerical_identity = identity ? std::string_view(identity) : std::string_view();
    q.shape = a8::DownShape{hidden, intermediate, experts, top_k};
    q.weight_type = weight_type; q.swiglu_limit = limit;
    a8::DeviceBytes v[9];
    for (int i = 0; i < 9; ++i) v[i] = a8::DeviceBytes{static_cast<std::uintptr_t>(views[2 * i]), views[2 * i + 1]};
    const a8::DownBindings b{v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], v[8]};
    return guarded([&] { a8::validate_down(q, b); });
}
// The union rows form: validate_union / validate_down_union (src/moe_q4k_a8_contract.cpp:373-405, src/moe_a8_down_contract.cpp:83-113)
// with the plan view as a tenth {address, bytes} pair, and expert_union::build (include/strix/moe/expert_union.hpp:34-57), whose
// entries land in `entries` as 12 bytes each (at most 128); returns their number, -1 when build() refuses the ids.
int ref_a8_validate_union(int enabled, const char* identity, int input_fp32, std::uint32_t hidden, std::uint32_t rows, std::uint32_t experts,
                          std::uint32_t top_k, std::uint32_t logical_rows, std::uint32_t gate_type, std::uint32_t up_type, int fused, float limit,
                          const std::uint64_t* views) {
    a8::Request q;
    q.enabled = enabled != 0; q.approved_numerical_identity = identity ? std::string_view(identity) : std::string_view();
    q.input = input_fp32 ? a8::InputKind::fp32 : a8::InputKind::bf16;
    q.shape = a8::Shape{hidden, rows, experts, top_k, logical_rows};
    q.gate_type = gate_type; q.up_type = up_type; q.fused_gate_up = fused != 0; q.swiglu_limit = limit;
    a8::DeviceBytes v[10];
    for (int i = 0; i < 10; ++i) v[i] = a8::DeviceBytes{static_cast<std::uintptr_t>(views[2 * i]), views[2 * i + 1]};
    const a8::Bindings b{v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], v[8]};
    return guarded([&] { a8::validate_union(q, b, v[9]); });
}
int ref_a8_validate_down_union(int enabled, const char* identity, std::uint32_t hidden, std::uint32_t intermediate, std::uint32_t experts,
                               std::uint32_t top_k, std::uint32_t weight_type, float limit, std::uint32_t rows, const std::uint64_t* views) {
    a8::DownRequest q;
    q.enabled = enabled != 0; q.approved_numerical_identity = identity ? std::string_view(identity) : std::string_view();
    q.shape = a8::DownShape{hidden, intermediate, experts, top_k};
    q.weight_type = weight_type; q.swiglu_limit = limit;
    a8::DeviceBytes v[10];
    for (int i = 0; i < 10; ++i) v[i] = a8::DeviceBytes{static_cast<std::uintptr_t>(views[2 * i]), views[2 * i + 1]};
    const a8::DownBindings b{v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], v[8]};
    return guarded([&] { a8::validate_down_union(q, b, rows, v[9]); });
}
int ref_expert_union_build(const std::uint32_t* ids, std::uint32_t rows, std::uint32_t top_k, std::uint32_t experts, unsigned char* entries) {
    int count = -1;
    guarded([&] {
        const auto plan = strix::moe::expert_union::build(std::span<const std::uint32_t>(ids, std::size_t{rows} * top_k), rows, top_k, experts);
        std::memcpy(entries, plan.data(), plan.size() * sizeof(strix::moe::expert_union::Entry));
        count = static_cast<int>(plan.size());
    });
    return count;
}
const char* ref_a8_identity(std::uint32_t type, int down) {
    static std::string held;
    try { held = std::string(down ? a8::down_numerical_identity(type) : a8::numerical_identity_for_gate_type(type)); } catch (const std::exception&) { held.clear(); }
    return held.c_str();
}

void ref_swiglu_clamp(float gate, float up, float limit, float* gate_out, float* up_out) {
    const auto c = strix::moe::swiglu_clamp(gate, up, limit);
    *gate_out = c.gate; *up_out = c.up;
}
int ref_combine_fma(std::uint32_t rows, std::uint32_t top_k, std::uint32_t width, const float* w, const float* eo,
                    const float* base, float* y) {
    return guarded([&] {
        const std::size_t n = std::size_t{rows} * width;
        strix::moe::combine_ref(strix::moe::CombineForm::fma_f32, rows, top_k, width, std::span<const float>(w, std::size_t{rows} * top_k),
                                std::span<const float>(eo, n * top_k), std::span<const float>(base, n), std::span<float>(y, n));
    });
}
// w and / or base may be null (unit weights, no base): the bf16-steps form of the same function
int ref_combine_bf16_steps(std::uint32_t rows, std::uint32_t top_k, std::uint32_t width, const float* w, const float* eo,
                           const float* base, float* y) {
    return guarded([&] {
        const std::size_t n = std::size_t{rows} * width;
        strix::moe::combine_ref(strix::moe::CombineForm::bf16_steps, rows, top_k, width,
                                w ? std::span<const float>(w, std::size_t{rows} * top_k) : std::span<const float>(),
                                std::span<const float>(eo, n * top_k), base ? std::span<const float>(base, n) : std::span<const float>(),
                                std::span<float>(y, n));
    });
}
float ref_combine_round_bf16(float x) { return strix::moe::combine_round_bf16(x); }

}  // extern "C"
