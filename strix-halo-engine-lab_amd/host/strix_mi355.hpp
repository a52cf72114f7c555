// Header-only C++ mirror of the engine-side interfaces this library replaces, over the C ABI in mi355_strix.h: the
// reference's struct and function names, argument order and error behaviour, so that a call site written against the
// reference compiles against this namespace after the changes listed here and nothing else:
//   * namespace strix::mi355 in the place of strix; device memory everywhere (the CPU interfaces below take device pointers);
//   * a stream argument where the reference has a thread pool or a cudaStream_t (mi355_stream = hipStream_t as void*);
//   * qwen_moe::Rows carries the model geometry (the reference twin fixes it at compile time, include/strix/cuda/qwen_moe.hpp:27),
//     its Csr views are this library's plan words, and enqueue_project / enqueue take no amdmath::Tables (the exp kind is in Weights);
//   * expert::Executor is constructed with its capacity (max assignments, max ffn) instead of a thread count.
// Interfaces:
//   cpu::Q8a8View / Stream / Kernels            src/cpu/core/backend.hpp:52-73
//   weight::Candidate / Plan / WeightView / KernelArguments / enqueue / enqueue_dense   include/strix/weight/resolve.hpp:67-84,
//                                                                                     src/cpu/weight/registry.cpp:11-63
//   weight::RuntimeCallbacks / ExecutionContext / Retirement / Hardware / RuntimeAdapter, bind_runtime, enqueue(.., context)
//                                                                                     include/strix/weight/cache.hpp:6-33, runtime.hpp:5-13,
//                                                                                     src/weight/cache.cpp:192-200 (the HIP binding:
//                                                                                     strix_mi355_runtime.hpp, bind_native_runtime)
//   moe_q4k_a8::Request .. Bindings, validate, enqueue_probe                          include/strix/moe_q4k_a8_contract.hpp:101-122,
//                                                                                     include/strix/hip_moe_q4k_a8_probe.hpp:12
//   moe_q4k_a8::DownRequest .. DownBindings, validate_down, enqueue_down_*, SlotMergeTail   include/strix/moe_a8_down_contract.hpp:39-54,
//                                                                                     include/strix/hip_moe_a8_down.hpp:11-30
//   qwen_moe::Strided / Rows / Weights, enqueue_prologue .. enqueue_commit, enqueue   include/strix/cuda/qwen_moe.hpp:34-110
//   expert::LayerWeights / RowA8 / Assignment / Job / Executor                        src/cpu/core/routed_expert.hpp:28-95
//   moe_q4k_a8::enqueue_serial_prologue_probe, enqueue_quantize_only                  include/strix/hip_moe_q4k_a8_probe.hpp:20-24
//   moe::CombineForm, moe_core::enqueue_combine, enqueue_combine_rounded_eo           include/strix/moe/combine.hpp:13,
//                                                                                     src/moe_core/route_wave_kernel.hpp:138-160
//   moe_route::enqueue                                                                the policy of include/strix/moe_core/route_policy.hpp
// Admission failures throw std::invalid_argument before anything is enqueued, HIP failures throw std::runtime_error, as the
// reference's check / hip_check do. Nothing here allocates (Executor's constructor aside) or synchronises.
#pragma once
#include <cstddef>
#include <cstdint>
#include <functional>
#include <memory>
#include <limits>
#include <stdexcept>
#include <string>
#include <string_view>
#include <type_traits>
#include <vector>

#include "mi355_strix.h"

namespace strix::mi355 {

inline void check(std::int32_t rc) {
    if (rc == MI355_OK) return;
    const std::string why = mi355_last_error();
    if (rc == MI355_E_INVALID_ARGUMENT || rc == MI355_E_UNSUPPORTED) throw std::invalid_argument(why);
    throw std::runtime_error(why);
}

// ---------------------------------------------------------------------------------------------- dense kernel table
namespace cpu {
using Q8a8View = mi355_q8a8_view;                       // field for field strix::cpu::Q8a8View
struct Stream { mi355_stream stream = nullptr; };       // the reference's Stream carries the worker pool; here the HIP stream
// The kernel table: the three entries of strix::cpu::Kernels with their signatures. quantize_a8 and gemv_q8_0_a8 throw
// std::invalid_argument for a width / in not divisible by 32 before writing any output; zero width is allowed.
struct Kernels {
    void (*quantize_a8)(const float* x, std::size_t width, std::int8_t* codes, float* deltas, std::int32_t* sums);
    void (*gemv_q8_0_a8)(const Q8a8View& v, const Stream& s);
    void (*rmsnorm_f32)(const float* x, const float* w, unsigned n, float eps, float* y, unsigned rows, const Stream& s);
};
inline const Kernels& mi355_kernels() noexcept {
    static const Kernels table{
        [](const float* x, std::size_t width, std::int8_t* codes, float* deltas, std::int32_t* sums) {
            check(mi355_quantize_a8(x, MI355_INPUT_F32, 1, static_cast<std::uint32_t>(width), width * sizeof(float), codes, deltas, sums, nullptr, nullptr));
        },
        [](const Q8a8View& v, const Stream& s) { check(mi355_gemv_q8_0_a8(&v, s.stream)); },
        [](const float* x, const float* w, unsigned n, float eps, float* y, unsigned rows, const Stream& s) {
            check(mi355_rmsnorm_f32(x, w, n, eps, y, rows, s.stream));
        }};
    return table;
}
}  // namespace cpu

// ---------------------------------------------------------------------------------------------- typed weight-operator registry
// The checked launch envelope of the reference's weight registry (Candidate / Plan / WeightView / KernelArguments / enqueue,
// include/strix/weight/types.hpp:18-64, include/strix/weight/resolve.hpp:67-84) with the one registration the CPU backend
// makes, the raw Q8_0 tree32 product (src/cpu/weight/registry.cpp:11-63, src/cpu/weight/source.hpp:17-38): the same kernel id,
// storage / arithmetic / image ids, schema and ABI revision, and the same refusals in the same order (a plan that does not
// select this kernel and arithmetic: unsupported_arithmetic; an envelope of another schema, revision or size: malformed; a
// null operand: malformed; dimensions or strides: unsupported_shape), Status instead of exceptions. The payload is device
// memory; output replaces view.out as in the reference's dispatch.
namespace weight {
using TensorId = std::uint64_t;
using KernelId = std::uint64_t;
struct Id { std::string_view name; std::uint32_t revision; };
inline bool operator==(Id a, Id b) noexcept { return a.revision == b.revision && a.name == b.name; }
using FormatId = Id; using ArithmeticId = Id; using ImageId = Id;
enum class Backend : std::uint8_t { hip, cuda, cpu, intel };
enum class Exactness : std::uint8_t { legacy_bitwise, operand_exact, fast };
enum class Strategy : std::uint8_t { native, staged, converted, onfly };
enum class Error : std::uint8_t { ok, unknown_format, malformed, unsupported_role, unsupported_shape, unsupported_backend, unsupported_arithmetic,
                                  unavailable_isa, memory_budget, unqualified, stale_source, device_failure };
struct Status { Error code; std::string detail; explicit operator bool() const { return code == Error::ok; } };
struct Shape { std::uint64_t dims[4]; std::uint8_t rank; };
struct WeightView { TensorId tensor; FormatId storage; Shape shape; const std::uint8_t* payload; std::uint64_t payload_bytes; };   // payload: device memory
struct Candidate { KernelId kernel; FormatId storage; ArithmeticId arithmetic; ImageId image; Backend backend; Strategy strategy; Exactness exactness; };
struct Plan { Candidate selected; std::uint64_t workspace_bytes = 0; };
struct KernelArguments { KernelId schema; std::uint32_t abi_revision; const void* data; std::size_t bytes; };
// What a backend installs under the registry (include/strix/weight/cache.hpp:6-33, include/strix/weight/runtime.hpp:5-13,
// include/strix/weight/resolve.hpp:7-15): allocation, events, the upload of a weight image, deferred reclamation and the typed
// launch. strix_mi355_runtime.hpp binds them to HIP and to this library (bind_native_runtime).
struct Retirement {
    std::vector<void*> events;                 // last-use events: the allocation is reclaimed after all of them
    std::vector<void*> unresolved_streams;     // streams whose last use could not be recorded: drained before reclamation
    std::shared_ptr<void> reservation;         // released only after the allocation is actually freed
};
struct ExecutionContext;
struct RuntimeCallbacks {
    std::function<Status(std::uint64_t, void*&)> allocate;
    std::function<void(void*)> free;
    std::function<Status(ExecutionContext&, void*&)> record_event;
    std::function<Status(ExecutionContext&, void*)> wait_event;
    std::function<bool(void*)> event_complete;
    std::function<void(void*)> destroy_event;
    std::function<Status(const WeightView&, const Plan&, void*, ExecutionContext&)> convert;
    std::function<void(void*, Retirement, ExecutionContext)> retire;       // takes the allocation, its fences and its budget; must not throw
    std::function<Status(const Plan&, const WeightView&, const KernelArguments&, void*, void*, std::size_t, ExecutionContext&)> enqueue;
};
struct ExecutionContext {
    Backend backend = Backend::cpu;
    void* stream = nullptr;
    std::uint32_t device_index = 0;
    std::shared_ptr<const RuntimeCallbacks> callbacks;
};
struct Hardware {
    Backend backend; std::string arch, compiler_id, device_class;
    std::uint64_t isa_mask, free_bytes, cache_budget_bytes;
    std::uint32_t registers_per_sm, registers_per_thread_limit;
    std::uint32_t shared_bytes_per_sm, warp_or_wave;
    double memory_bytes_per_second, lookup_per_second, dot4_per_second;
    double valu_ops_per_second, matrix_ops_per_second;
    bool valu_matrix_serialize;
};
struct RuntimeAdapter {
    std::shared_ptr<const RuntimeCallbacks> callbacks;
    std::function<Status(std::uint32_t, Hardware&)> query_hardware;
};
inline std::string current_compiler_id() {       // src/weight/runtime.cpp:3-13
#if defined(__clang__)
    return "clang/" __clang_version__;
#elif defined(__GNUC__)
    return "gcc/" __VERSION__;
#else
    return "unknown-compiler";
#endif
}
// src/weight/runtime.cpp:15-24: the same refusals in the same order
inline Status bind_runtime(Backend backend, const RuntimeAdapter& adapter, void* stream, std::uint32_t device, ExecutionContext& context, Hardware& hardware) {
    if (!adapter.callbacks || !adapter.query_hardware) return {Error::unsupported_backend, "backend runtime not registered"};
    Hardware h{};
    Status status = adapter.query_hardware(device, h);
    if (!status) return status;
    if (h.backend != backend) return {Error::unsupported_backend, "capability query returned another backend"};
    context = {backend, stream, device, adapter.callbacks};
    hardware = std::move(h);
    return {Error::ok, {}};
}
template <class Args> struct ArgumentTraits;
template <class Args> KernelArguments arguments(Args& args) {
    using Type = std::remove_cv_t<Args>;
    static_assert(std::is_standard_layout_v<Type> && std::is_trivially_copyable_v<Type>);
    return {ArgumentTraits<Type>::schema, ArgumentTraits<Type>::abi_revision, &args, sizeof(Type)};
}
template <class Args> KernelArguments arguments(const Args&&) = delete;

inline constexpr KernelId q8_tree32_kernel = 0x43505501;
struct DenseArguments { cpu::Q8a8View view; cpu::Stream stream; };
template <> struct ArgumentTraits<DenseArguments> {
    static constexpr KernelId schema = q8_tree32_kernel;
    static constexpr std::uint32_t abi_revision = 2;
};
inline const Candidate* candidates(std::size_t& count) noexcept {
    static const Candidate entries[] = {{q8_tree32_kernel, {"gguf.q8_0", 1}, {"cpu-q8a8-tree32", 1}, {"cpu.q8-raw", 1}, Backend::hip, Strategy::native,
                                         Exactness::legacy_bitwise}};
    count = 1;
    return entries;
}
inline Status validate_view(const cpu::Q8a8View& view) {
    if (!view.weight || !view.codes || !view.deltas || !view.out) return {Error::malformed, "Q8 launch has null operand"};
    if (!view.in || !view.count || !view.rows || view.in % 32U || view.x_stride % 32U || view.x_stride < view.in ||
        static_cast<std::uint64_t>(view.in / 32U) * 34U > view.row_bytes || view.out_stride < view.count)
        return {Error::unsupported_shape, "Q8 launch dimensions/strides"};
    return {Error::ok, {}};
}
// weight: [count][in] Q8_0 rows (dims fastest first: in, count)
inline Status validate_q8_shape(const WeightView& weight, std::uint64_t count, std::uint64_t in) {
    if (!(weight.storage == FormatId{"gguf.q8_0", 1})) return {Error::unknown_format, "weight is not raw Q8_0"};
    if (weight.shape.rank != 2 || weight.shape.dims[0] != in || weight.shape.dims[1] != count) return {Error::unsupported_shape, "Q8 weight shape differs from the launch"};
    if (!weight.payload || weight.payload_bytes < count * (in / 32U) * 34U) return {Error::malformed, "Q8 weight payload shorter than its shape"};
    return {Error::ok, {}};
}
// The launch through a bound context (src/weight/cache.cpp:192-200): backend, storage, workspace, envelope, launcher - refused
// in that order - then the backend's own enqueue callback.
inline Status enqueue(const Plan& plan, const WeightView& view, const KernelArguments& args, void* output, void* workspace, std::size_t workspace_bytes,
                      ExecutionContext& context) {
    if (context.backend != plan.selected.backend) return {Error::unsupported_backend, "enqueue context backend differs"};
    if (!(view.storage == plan.selected.storage)) return {Error::unknown_format, "enqueue storage differs"};
    if (workspace_bytes < plan.workspace_bytes || (plan.workspace_bytes && !workspace)) return {Error::memory_budget, "workspace missing or too short"};
    if (!args.data || !args.bytes || !args.schema || !args.abi_revision || !output) return {Error::malformed, "invalid typed argument envelope"};
    if (!context.callbacks || !context.callbacks->enqueue) return {Error::unsupported_arithmetic, "backend has no registered launcher"};
    return context.callbacks->enqueue(plan, view, args, output, workspace, workspace_bytes, context);
}
// The registration's own dispatch (src/cpu/weight/registry.cpp:11-32): what the enqueue callback of a bound context calls.
inline Status enqueue(const Plan& plan, const WeightView& weight, const KernelArguments& envelope, void* output, void* /*workspace*/, std::size_t /*workspace_bytes*/) {
    if (plan.selected.kernel != q8_tree32_kernel || !(plan.selected.arithmetic == ArithmeticId{"cpu-q8a8-tree32", 1}) || plan.selected.strategy != Strategy::native)
        return {Error::unsupported_arithmetic, "the registry only provides the raw Q8_0 tree32 incumbent"};
    if (envelope.schema != q8_tree32_kernel || envelope.abi_revision != 2 || envelope.bytes != sizeof(DenseArguments) || !envelope.data)
        return {Error::malformed, "Q8 typed launch schema/ABI"};
    const DenseArguments& args = *static_cast<const DenseArguments*>(envelope.data);
    cpu::Q8a8View view = args.view;
    view.out = static_cast<float*>(output);
    view.weight = weight.payload;
    Status status = validate_view(view);
    if (!status) return status;
    status = validate_q8_shape(weight, view.count, view.in);
    if (!status) return status;
    const std::int32_t rc = mi355_gemv_q8_0_a8(&view, args.stream.stream);
    if (rc != MI355_OK) return {rc == MI355_E_HIP ? Error::device_failure : Error::unsupported_shape, mi355_last_error()};
    return {Error::ok, {}};
}
// A context that carries only the launcher (src/cpu/weight/registry.cpp:49-59); strix_mi355_runtime.hpp's bind_native_runtime
// gives one with allocation, events, upload and retirement as well.
inline ExecutionContext execution_context() {
    static const std::shared_ptr<const RuntimeCallbacks> callbacks = [] {
        auto result = std::make_shared<RuntimeCallbacks>();
        result->enqueue = [](const Plan& plan, const WeightView& weight, const KernelArguments& args, void* output, void* workspace, std::size_t bytes, ExecutionContext&) {
            return enqueue(plan, weight, args, output, workspace, bytes);
        };
        return result;
    }();
    return {Backend::hip, nullptr, 0, callbacks};
}
inline Status enqueue_dense(const WeightView& weight, const DenseArguments& args) {
    std::size_t n;
    Plan plan{candidates(n)[0]};
    ExecutionContext context = execution_context();
    DenseArguments launch = args;
    return enqueue(plan, weight, arguments(launch), args.view.out, nullptr, 0, context);
}
}  // namespace weight

// ---------------------------------------------------------------------------------------------- expert union of a verify window
// include/strix/moe/expert_union.hpp: the plan layout the union entry points of the A8 contract share, and its host builder
// (the reference of the device builder inside enqueue_probe_union).
namespace moe::expert_union {
inline constexpr std::uint32_t max_rows = MI355_UNION_MAX_ROWS, max_top_k = MI355_UNION_MAX_TOP_K, max_assignments = max_rows * max_top_k;
inline constexpr std::uint8_t no_slot = 0xFFU;
struct Header { std::uint32_t count = 0, rows = 0, top_k = 0, reserved = 0; };
struct Entry { std::uint32_t expert; std::uint8_t slot[max_rows]; };
static_assert(sizeof(Header) == 16U && sizeof(Entry) == 12U);
inline constexpr std::uint64_t plan_bytes = sizeof(Header) + std::uint64_t{max_assignments} * sizeof(Entry);
static_assert(plan_bytes == MI355_UNION_PLAN_BYTES);
[[nodiscard]] constexpr bool admits(std::uint32_t rows, std::uint32_t top_k) noexcept { return rows >= 1U && rows <= max_rows && top_k >= 1U && top_k <= max_top_k; }
// ids: rows x top_k expert ids, row-major. std::invalid_argument on a shape outside admits(), an id >= experts or an id named
// twice by one row.
[[nodiscard]] inline std::vector<Entry> build(const std::uint32_t* ids, std::size_t count, std::uint32_t rows, std::uint32_t top_k, std::uint32_t experts) {
    if (!admits(rows, top_k) || count != std::size_t{rows} * top_k) throw std::invalid_argument("expert union: rows <= 8, top_k <= 16 and rows x top_k ids required");
    std::vector<Entry> plan;
    for (std::size_t a = 0; a < count; ++a) {
        const std::uint32_t e = ids[a], row = static_cast<std::uint32_t>(a / top_k);
        if (e >= experts) throw std::invalid_argument("expert union: expert id out of range");
        Entry* held = nullptr;
        for (Entry& entry : plan)
            if (entry.expert == e) { held = &entry; break; }
        if (!held) {
            Entry fresh;
            fresh.expert = e;
            for (std::uint8_t& slot : fresh.slot) slot = no_slot;
            plan.push_back(fresh);
            held = &plan.back();
        }
        if (held->slot[row] != no_slot) throw std::invalid_argument("expert union: expert repeated within one row");
        held->slot[row] = static_cast<std::uint8_t>(a % top_k);
    }
    return plan;
}
}  // namespace moe::expert_union

// ---------------------------------------------------------------------------------------------- A8 request / bindings
namespace moe_q4k_a8 {
inline constexpr float kSwigluNoClamp = std::numeric_limits<float>::infinity();
inline constexpr unsigned invalid_route = 1U, nonfinite_activation = 2U, invalid_delta = 4U;
inline constexpr std::uint32_t down_invalid_route = 1, down_nonfinite_activation = 8, down_aggregate_error = 16;

enum class InputKind { bf16, fp32, fp16 };              // the reference has bf16 and fp32
struct Shape { std::uint32_t hidden = 256, rows = 32, experts = 1, top_k = 1, logical_rows = 1; };
struct Request {
    bool enabled = false;
    std::string_view approved_numerical_identity;
    InputKind input = InputKind::bf16;
    Shape shape;
    std::uint32_t gate_type = 12, up_type = 12;
    bool fused_gate_up = false;
    float swiglu_limit = kSwigluNoClamp;
};
struct DeviceBytes { std::uintptr_t address = 0; std::uint64_t bytes = 0; };
struct Bindings { DeviceBytes input, gate, up, routes, codes, deltas, sums, status, output; };

[[nodiscard]] inline std::string_view numerical_identity_for_gate_type(std::uint32_t gate_type) {
    const char* id = mi355_numerical_identity(gate_type, 0);
    if (!id[0]) throw std::invalid_argument("A8 gate/up requires type12 or type13");
    return id;
}
[[nodiscard]] inline std::string_view down_numerical_identity(std::uint32_t weight_type) {
    const char* id = mi355_numerical_identity(weight_type, 1);
    if (!id[0]) throw std::invalid_argument("A8 down weights must be type 7, 8, 12 or 14");
    return id;
}

namespace detail {
inline mi355_device_bytes c(const DeviceBytes& v) { return mi355_device_bytes{v.address, v.bytes}; }
struct CRequest { std::string identity; mi355_a8_request q; };
inline void fill(const Request& r, CRequest& out) {
    out.identity = std::string(r.approved_numerical_identity);
    out.q = mi355_a8_request{r.enabled ? 1U : 0U, out.identity.c_str(),
                             r.input == InputKind::bf16 ? MI355_INPUT_BF16 : r.input == InputKind::fp32 ? MI355_INPUT_F32 : MI355_INPUT_F16,
                             mi355_a8_shape{r.shape.hidden, r.shape.rows, r.shape.experts, r.shape.top_k, r.shape.logical_rows},
                             r.gate_type, r.up_type, r.fused_gate_up ? 1U : 0U, r.swiglu_limit};
}
inline mi355_a8_bindings c(const Bindings& b) {
    return mi355_a8_bindings{c(b.input), c(b.gate), c(b.up), c(b.routes), c(b.codes), c(b.deltas), c(b.sums), c(b.status), c(b.output)};
}
}  // namespace detail

// Pure host admission; no allocation, HIP call or buffer mutation.
inline void validate(const Request& request, const Bindings& bindings) {
    detail::CRequest q; detail::fill(request, q);
    const mi355_a8_bindings b = detail::c(bindings);
    check(mi355_a8_validate(&q.q, &b));
}
inline void enqueue_probe(const Request& request, const Bindings& bindings, mi355_stream stream = nullptr) {
    detail::CRequest q; detail::fill(request, q);
    const mi355_a8_bindings b = detail::c(bindings);
    check(mi355_a8_enqueue_probe(&q.q, &b, stream));
}

// include/strix/hip_moe_q4k_a8_probe.hpp:20-23: the serial row's clear + route / route-weight check + quantiser in one workgroup,
// status overwritten, then the projection
inline void enqueue_serial_prologue_probe(const Request& request, const Bindings& bindings, float* clear, unsigned clear_words,
                                          const float* route_weights, mi355_stream stream) {
    detail::CRequest q; detail::fill(request, q);
    const mi355_a8_bindings b = detail::c(bindings);
    check(mi355_a8_enqueue_serial_prologue_probe(&q.q, &b, clear, clear_words, route_weights, stream));
}
// include/strix/hip_moe_q4k_a8_probe.hpp:24: route check + quantiser, no projection
inline void enqueue_quantize_only(const Request& request, const Bindings& bindings, mi355_stream stream) {
    detail::CRequest q; detail::fill(request, q);
    const mi355_a8_bindings b = detail::c(bindings);
    check(mi355_a8_enqueue_quantize_only(&q.q, &b, stream));
}

// Union rows form (include/strix/moe_q4k_a8_contract.hpp:123-132, src/hip_moe_q4k_a8_probe.hip:1172-1191): shape.logical_rows = R
// (1..8); the per-row views are R contiguous single-row extents; plan = moe::expert_union::plan_bytes, written by the probe.
inline void validate_union(const Request& request, const Bindings& bindings, DeviceBytes plan) {
    detail::CRequest q; detail::fill(request, q);
    const mi355_a8_bindings b = detail::c(bindings);
    check(mi355_a8_validate_union(&q.q, &b, detail::c(plan)));
}
inline void enqueue_probe_union(const Request& request, const Bindings& bindings, DeviceBytes plan, mi355_stream stream) {
    detail::CRequest q; detail::fill(request, q);
    const mi355_a8_bindings b = detail::c(bindings);
    check(mi355_a8_enqueue_probe_union(&q.q, &b, detail::c(plan), stream));
}

struct DownShape { std::uint32_t hidden = 0, intermediate = 0, experts = 0, top_k = 0; };
struct DownRequest {
    bool enabled = false;
    std::string_view approved_numerical_identity;
    DownShape shape;
    std::uint32_t weight_type = 7;
    float swiglu_limit = kSwigluNoClamp;
};
struct DownBindings { DeviceBytes intermediates, weights, routes, codes, deltas, sums, rawdots, status, aggregate_status; };
struct SlotMergeTail {
    std::uint32_t* tickets = nullptr;
    const float* route_weights = nullptr;
    float* accumulation = nullptr;
    void* output = nullptr;
    bool output_bf16 = false, bf16_commit = false;
    void* record = nullptr;  // DeferredMoeFirstError {domain, bits}
    std::uint32_t domain = 0;
};
namespace detail {
struct CDownRequest { std::string identity; mi355_a8_down_request q; };
inline void fill(const DownRequest& r, CDownRequest& out) {
    out.identity = std::string(r.approved_numerical_identity);
    out.q = mi355_a8_down_request{r.enabled ? 1U : 0U, out.identity.c_str(),
                                  mi355_a8_down_shape{r.shape.hidden, r.shape.intermediate, r.shape.experts, r.shape.top_k}, r.weight_type, r.swiglu_limit};
}
inline mi355_a8_down_bindings c(const DownBindings& b) {
    return mi355_a8_down_bindings{c(b.intermediates), c(b.weights), c(b.routes), c(b.codes), c(b.deltas), c(b.sums), c(b.rawdots), c(b.status),
                                  c(b.aggregate_status)};
}
}  // namespace detail
inline void validate_down(const DownRequest& request, const DownBindings& bindings) {
    detail::CDownRequest q; detail::fill(request, q);
    const mi355_a8_down_bindings b = detail::c(bindings);
    check(mi355_a8_validate_down(&q.q, &b, 1));
}
// The SiLU's expf is the gfx1151 device function's host twin, as in the reference's kernels.
inline void enqueue_down_activation_quantize(const DownRequest& request, const DownBindings& bindings, mi355_stream stream) {
    detail::CDownRequest q; detail::fill(request, q);
    const mi355_a8_down_bindings b = detail::c(bindings);
    check(mi355_a8_enqueue_down_activation_quantize(&q.q, &b, 1, MI355_EXP_GFX1151, stream));
}
inline void enqueue_down_rawdots(const DownRequest& request, const DownBindings& bindings, mi355_stream stream) {
    detail::CDownRequest q; detail::fill(request, q);
    const mi355_a8_down_bindings b = detail::c(bindings);
    check(mi355_a8_enqueue_down_rawdots(&q.q, &b, 1, stream));
}
inline void enqueue_down_rawdots(const DownRequest& request, const DownBindings& bindings, const SlotMergeTail& tail, mi355_stream stream) {
    detail::CDownRequest q; detail::fill(request, q);
    const mi355_a8_down_bindings b = detail::c(bindings);
    const mi355_slot_merge_tail t{tail.tickets, tail.route_weights, tail.accumulation, tail.output, tail.output_bf16 ? 1U : 0U, tail.bf16_commit ? 1U : 0U,
                                  tail.record, tail.domain};
    check(mi355_a8_enqueue_down_rawdots_merge(&q.q, &b, &t, stream));
}
// Union rows form of the K-quant down class (include/strix/moe_a8_down_contract.hpp:57-60, src/hip_moe_q4k_a8_probe.hip:1192-1221).
inline void validate_down_union(const DownRequest& request, const DownBindings& bindings, std::uint32_t rows, DeviceBytes plan) {
    detail::CDownRequest q; detail::fill(request, q);
    const mi355_a8_down_bindings b = detail::c(bindings);
    check(mi355_a8_validate_down_union(&q.q, &b, rows, detail::c(plan)));
}
inline void enqueue_down_activation_quantize_union(const DownRequest& request, const DownBindings& bindings, std::uint32_t rows, DeviceBytes plan, mi355_stream stream) {
    detail::CDownRequest q; detail::fill(request, q);
    const mi355_a8_down_bindings b = detail::c(bindings);
    check(mi355_a8_enqueue_down_activation_quantize_union(&q.q, &b, rows, detail::c(plan), MI355_EXP_GFX1151, stream));
}
inline void enqueue_down_rawdots_union(const DownRequest& request, const DownBindings& bindings, std::uint32_t rows, DeviceBytes plan, mi355_stream stream) {
    detail::CDownRequest q; detail::fill(request, q);
    const mi355_a8_down_bindings b = detail::c(bindings);
    check(mi355_a8_enqueue_down_rawdots_union(&q.q, &b, rows, detail::c(plan), stream));
}
}  // namespace moe_q4k_a8

// ---------------------------------------------------------------------------------------------- strided multi-row layer
namespace qwen_moe {
inline constexpr std::uint32_t invalid_route = 1, nonfinite_activation = 2, invalid_delta = 4, projection_nonfinite = 8;
inline constexpr std::uint32_t type_q5_1 = 7, type_q8_0 = 8, type_q4_k = 12, type_q5_k = 13, type_q6_k = 14;
// Row r of a view lives at base + r * stride (bytes). Every base and stride must be 16-byte aligned (routes, route weights
// and status: 4).
template <class T> struct Strided { T* base = nullptr; std::uint64_t stride = 0; };
struct Geometry { std::uint32_t hidden = 0, ffn = 0, experts = 0, top_k = 0; };
struct Csr { std::uint32_t* plan = nullptr; std::uint32_t* summary = nullptr; };   // plan: mi355_moe_plan_words(); summary: one word (the job status)
struct Rows {
    Strided<const std::uint16_t> input;        // BF16 [hidden]
    Strided<const std::uint32_t> routes;       // [top_k]
    Strided<const float> route_weights;        // [top_k]
    Strided<std::int8_t> codes;                // [hidden]
    Strided<float> deltas;                     // [hidden / 32]
    Strided<std::int32_t> sums;                // [hidden / 32]
    Strided<std::uint32_t> status;             // [1]
    Strided<float> intermediates;              // [top_k * 2 * ffn]: h | u per slot; base may be null (not written)
    Strided<float> accumulation;               // [clear_words >= hidden]: zeroed by the prologue, merge result
    Strided<std::int8_t> down_codes;           // [top_k * ffn]
    Strided<float> down_deltas;                // [top_k * ffn / 32]
    Strided<std::int32_t> down_sums;           // [top_k * ffn / 32]
    Strided<float> rawdots;                    // [top_k * hidden]
    Strided<std::uint16_t> output;             // BF16 [hidden]
    Csr csr;
    Geometry geometry;
};
struct Weights {
    std::uint32_t gate_type = type_q4_k;       // 12 or 13 (gate and up share it)
    const std::uint8_t* gate = nullptr;        // [experts][ffn][hidden/256 blocks]
    const std::uint8_t* up = nullptr;
    std::uint32_t down_type = type_q5_1;       // 7, 8, 12 or 14
    const std::uint8_t* down = nullptr;        // [experts][hidden][ffn/32 blocks] (K-quants: ffn/256 super-blocks)
    std::uint32_t exp_kind = MI355_EXP_GFX1151;
    float swiglu_limit = std::numeric_limits<float>::infinity();
};
namespace detail {
template <class T> inline mi355_strided c(const Strided<T>& v) { return mi355_strided{const_cast<void*>(static_cast<const void*>(v.base)), v.stride}; }
inline mi355_moe_rows_strided c(const Rows& r) {
    mi355_moe_rows_strided v{};
    v.input = c(r.input); v.routes = c(r.routes); v.route_weights = c(r.route_weights); v.codes = c(r.codes); v.deltas = c(r.deltas); v.sums = c(r.sums);
    v.status = c(r.status); v.intermediates = c(r.intermediates); v.accumulation = c(r.accumulation); v.down_codes = c(r.down_codes);
    v.down_deltas = c(r.down_deltas); v.down_sums = c(r.down_sums); v.rawdots = c(r.rawdots); v.output = c(r.output);
    v.plan = r.csr.plan; v.job_status = r.csr.summary; v.input_kind = MI355_INPUT_BF16; v.output_kind = MI355_INPUT_BF16;
    return v;
}
// (the stages that read no weights are admitted on the geometry alone: default Weights)
inline mi355_moe_weights c(const Rows& r, const Weights& w) {
    mi355_moe_weights m{};
    m.hidden = r.geometry.hidden; m.ffn = r.geometry.ffn; m.experts = r.geometry.experts; m.top_k = r.geometry.top_k;
    m.gate_type = w.gate_type; m.down_type = w.down_type; m.gate = w.gate; m.up = w.up; m.down = w.down;
    m.exp_kind = w.exp_kind; m.swiglu_limit = w.swiglu_limit;
    return m;
}
}  // namespace detail
inline void enqueue_prologue(const Rows& r, std::uint32_t rows, std::uint32_t clear_words, mi355_stream s) {
    const auto v = detail::c(r); const auto m = detail::c(r, Weights{});
    check(mi355_moe_strided_enqueue_prologue(&m, &v, rows, clear_words, s));
}
inline void enqueue_csr(const Rows& r, std::uint32_t rows, mi355_stream s) {
    const auto v = detail::c(r); const auto m = detail::c(r, Weights{});
    check(mi355_moe_strided_enqueue_csr(&m, &v, rows, s));
}
inline void enqueue_project(const Rows& r, std::uint32_t rows, const Weights& w, mi355_stream s) {
    const auto v = detail::c(r); const auto m = detail::c(r, w);
    check(mi355_moe_strided_enqueue_project(&m, &v, rows, s));
}
inline void enqueue_down(const Rows& r, std::uint32_t rows, const Weights& w, mi355_stream s) {
    const auto v = detail::c(r); const auto m = detail::c(r, w);
    check(mi355_moe_strided_enqueue_down(&m, &v, rows, s));
}
inline void enqueue_merge(const Rows& r, std::uint32_t rows, mi355_stream s) {
    const auto v = detail::c(r); const auto m = detail::c(r, Weights{});
    check(mi355_moe_strided_enqueue_merge(&m, &v, rows, s));
}
// record: optional device DeferredMoeFirstError {domain, bits}; the domain is the reference's DeferredMoeDomain::q4k_a8 (2)
inline void enqueue_commit(const Rows& r, std::uint32_t rows, std::uint32_t* record, mi355_stream s) {
    const auto v = detail::c(r); const auto m = detail::c(r, Weights{});
    check(mi355_moe_strided_enqueue_commit(&m, &v, rows, record, 2U, s));
}
// prologue + csr + project + down + merge + commit
inline void enqueue(const Rows& r, std::uint32_t rows, std::uint32_t clear_words, const Weights& w, std::uint32_t* record, mi355_stream s) {
    const auto v = detail::c(r); const auto m = detail::c(r, w);
    check(mi355_moe_strided_enqueue(&m, &v, rows, clear_words, record, 2U, s));
}
}  // namespace qwen_moe

// ---------------------------------------------------------------------------------------------- host executor's job
namespace expert {
enum class GateFormat : std::uint8_t { q4_k, q5_k };
enum class DownFormat : std::uint8_t { q5_1, q8_0 };
struct Shape { std::uint32_t hidden = 0, ffn = 0; };
struct LayerWeights {
    const std::uint8_t* gate = nullptr;
    const std::uint8_t* up = nullptr;
    const std::uint8_t* down = nullptr;
    GateFormat gate_format = GateFormat::q4_k;
    DownFormat down_format = DownFormat::q5_1;
    Shape shape;
};
using RowA8 = mi355_row_a8;                    // codes, deltas, sums (device pointers)
using Assignment = mi355_expert_assignment;    // row, slot, expert
inline constexpr std::uint32_t kNonfinite = 1U;
struct Job {
    LayerWeights weights;
    const RowA8* rows = nullptr;               // device array, indexed by Assignment::row
    const Assignment* assignments = nullptr;   // device array
    std::uint32_t count = 0;
    float* rawdots = nullptr;                  // rawdots[row * rawdot_row_stride + slot * hidden + o]
    std::uint64_t rawdot_row_stride = 0;       // in floats
    std::uint32_t* status = nullptr;           // per row, OR-ed
};
class Executor {
public:
    Executor(std::uint32_t max_assignments, std::uint32_t max_ffn, std::uint32_t exp_kind = MI355_EXP_GFX1151)
        : handle_(mi355_executor_create(max_assignments, max_ffn, exp_kind)) {
        if (!handle_) throw std::invalid_argument(mi355_last_error());
    }
    ~Executor() { mi355_executor_destroy(handle_); }
    Executor(const Executor&) = delete;
    Executor& operator=(const Executor&) = delete;
    void run(const Job& job, mi355_stream stream = nullptr) {
        const mi355_expert_job j{mi355_layer_weights{job.weights.gate, job.weights.up, job.weights.down, static_cast<std::uint32_t>(job.weights.gate_format),
                                                     static_cast<std::uint32_t>(job.weights.down_format), job.weights.shape.hidden, job.weights.shape.ffn},
                                 job.rows, job.assignments, job.count, job.rawdots, job.rawdot_row_stride, job.status};
        check(mi355_executor_run(handle_, &j, stream));
    }
private:
    void* handle_;
};
}  // namespace expert

// ---------------------------------------------------------------------------------------------- combine
// include/strix/moe/combine.hpp:13 (CombineForm) and src/moe_core/route_wave_kernel.hpp:138-160 (enqueue_combine,
// enqueue_combine_rounded_eo); TopK and Width are template arguments there and stay so here.
namespace moe {
enum class CombineForm : std::uint8_t { fma_f32, bf16_steps };
}
namespace moe_core {
template <moe::CombineForm Form, unsigned TopK, unsigned Width>
void enqueue_combine(const float* w, const float* eo, const float* shared, float* y, unsigned rows, mi355_stream stream) {
    if (Form == moe::CombineForm::fma_f32 && (w == nullptr || shared == nullptr)) throw std::invalid_argument("moe combine: fma_f32 needs w and shared");
    check(mi355_moe_enqueue_combine(Form == moe::CombineForm::fma_f32 ? MI355_COMBINE_FMA_SLOT_ORDER : MI355_COMBINE_BF16_STEPS, rows, TopK, Width, w, eo,
                                    shared, y, 0U, stream));
}
template <moe::CombineForm Form, unsigned TopK, unsigned Width>
void enqueue_combine_rounded_eo(const float* w, const float* eo, const float* shared, float* y, unsigned rows, mi355_stream stream) {
    static_assert(Form == moe::CombineForm::bf16_steps, "moe combine: RoundEo is bound for bf16_steps only");
    check(mi355_moe_enqueue_combine(MI355_COMBINE_BF16_STEPS, rows, TopK, Width, w, eo, shared, y, 1U, stream));
}
}  // namespace moe_core

// ---------------------------------------------------------------------------------------------- router
namespace moe_route {
using Policy = mi355_route_policy;
inline void enqueue(const Policy& policy, const void* x, std::uint32_t input_kind, std::uint32_t rows, std::uint32_t hidden,
                    std::uint64_t x_stride_bytes, const float* router_weight, const float* logit_bias, std::uint32_t* ids,
                    float* weights, float* scores, mi355_stream stream) {
    check(mi355_moe_route(&policy, x, input_kind, rows, hidden, x_stride_bytes, router_weight, logit_bias, ids, weights, scores, stream));
}
}  // namespace moe_route

}  // namespace strix::mi355
