// The engine-side launcher of the routed-expert step over this library, as one translation unit written against the
// reference's REAL dispatch headers (include/strix/launch_dispatch.hpp, execution_runtime.hpp, dispatch_resources.hpp,
// moe_q4k_a8_runtime.hpp) and the C++ mirror (strix_mi355.hpp). It is what a maintainer adds to the reference tree as
// src/mi355_moe_experts_launcher.cpp. Here it is compiled, not run (tests/test_abi_cpu.py compiles it where the reference
// tree is present): the functions it declares from the reference (resolve_dispatch_*, build_runtime_workspace) live in the
// engine, not in this repository.
//
// The step it serves: SerialOp::moe_experts of one decode row (the reference's own launcher:
// src/hip_moe_experts_launcher.hip:1672-1760 prepare_moe_experts, :1387-1481 prepare_q4k_a8, :1483-1530 the enqueue order).
// reads = {hidden row, route indices, route weights}, writes = {the layer's output row}, temporaries = {the A8 workspace in the
// reference's own layout, RuntimeWorkspace}.
#include "strix/dispatch_resources.hpp"
#include "strix/execution_runtime.hpp"
#include "strix/launch_dispatch.hpp"
#include "strix/moe_q4k_a8_runtime.hpp"

#include "strix_mi355.hpp"

#include <cstdint>
#include <stdexcept>
#include <string>
#include <string_view>

namespace strix::mi355 {

struct MoeExpertsLauncherConfig {
    std::uint32_t hidden_size = 0, intermediate_size = 0, expert_count = 0, top_k = 0;
    bool bf16_activation = true;                       // storage of the hidden row and of the output row
    std::uint32_t gate_type = 12, down_type = 12;      // ggml ids: gate / up 12 | 13, down 7 | 8 | 12 | 14
    moe_q4k_a8::DeviceBytes gate, up, down;            // the layer's expert tensors in device memory (16-byte aligned)
    void* first_error_record = nullptr;                // device DeferredMoeFirstError {domain, bits}, or null
    mi355_stream stream = nullptr;                     // the engine's execution stream
};

namespace detail {
inline std::uint64_t fnv1a(std::string_view text, std::uint64_t h = 0xcbf29ce484222325ULL) {
    for (const char ch : text) h = (h ^ static_cast<unsigned char>(ch)) * 0x100000001b3ULL;
    return h;
}
}  // namespace detail

// ExecutionLaunchFunction (include/strix/launch_dispatch.hpp:15-17)
inline void launch_moe_experts(const ::strix::ExecutionDispatchContext& context, void* user_data) {
    namespace a8 = moe_q4k_a8;
    if (context.op != ::strix::SerialOp::moe_experts) throw std::invalid_argument("MI355 routed-expert launcher attached to wrong operator");
    if (context.reads.size() != 3 || context.writes.size() != 1 || context.temporaries.size() != 1)
        throw std::invalid_argument("MI355 routed experts expect hidden/routes/weights, one output and one temporary");
    if (context.logical_rows != 1 || context.request_concurrency != 1) throw std::invalid_argument("MI355 routed-expert launcher: one-row execution");
    if (user_data == nullptr) throw std::invalid_argument("MI355 routed experts require configuration");
    const auto& config = *static_cast<const MoeExpertsLauncherConfig*>(user_data);

    const ::strix::ExecutionBufferAddress hidden = ::strix::resolve_dispatch_read(context, 0);
    const ::strix::ExecutionBufferAddress route_indices = ::strix::resolve_dispatch_read(context, 1);
    const ::strix::ExecutionBufferAddress route_weights = ::strix::resolve_dispatch_read(context, 2);
    const ::strix::ExecutionBufferAddress output = ::strix::resolve_dispatch_write(context, 0);
    const ::strix::ExecutionBufferAddress temporary = ::strix::resolve_dispatch_temporary(context, 0);

    // the reference's own workspace layout with the integer down regions (rawdots, down codes / deltas / sums)
    const ::strix::moe_q4k_a8::RuntimeWorkspace layout = ::strix::moe_q4k_a8::build_runtime_workspace(
        config.hidden_size, config.intermediate_size, config.expert_count, config.top_k, false, true);
    if (temporary.bytes < layout.total_bytes) throw std::invalid_argument("MI355 routed experts: temporary is undersized");
    if (temporary.address % 256 != 0) throw std::invalid_argument("MI355 routed experts: temporary requires absolute 256-byte alignment");
    const std::uint64_t activation_bytes = config.bf16_activation ? 2U : 4U;
    if (hidden.bytes < config.hidden_size * activation_bytes || output.bytes < config.hidden_size * activation_bytes ||
        route_indices.bytes < config.top_k * sizeof(std::uint32_t) || route_weights.bytes < config.top_k * sizeof(float))
        throw std::invalid_argument("MI355 routed experts: a step buffer is undersized");
    const auto slice = [&](std::uint64_t offset, std::uint64_t bytes) {
        return a8::DeviceBytes{temporary.address + static_cast<std::uintptr_t>(offset), bytes};
    };

    a8::Request request;
    request.enabled = true;
    request.approved_numerical_identity = a8::numerical_identity_for_gate_type(config.gate_type);
    request.input = config.bf16_activation ? a8::InputKind::bf16 : a8::InputKind::fp32;
    request.shape = a8::Shape{config.hidden_size, config.intermediate_size, config.expert_count, config.top_k, 1};
    request.gate_type = request.up_type = config.gate_type;
    const a8::Bindings bindings{
        {hidden.address, config.hidden_size * activation_bytes}, config.gate, config.up,
        {route_indices.address, config.top_k * sizeof(std::uint32_t)},
        slice(layout.codes_offset, layout.codes_bytes), slice(layout.deltas_offset, layout.deltas_bytes),
        slice(layout.sums_offset, layout.sums_bytes), slice(layout.status_offset, 4), slice(layout.gate_up_offset, layout.gate_up_bytes)};
    a8::DownRequest down_request;
    down_request.enabled = true;
    down_request.approved_numerical_identity = a8::down_numerical_identity(config.down_type);
    down_request.shape = a8::DownShape{config.hidden_size, config.intermediate_size, config.expert_count, config.top_k};
    down_request.weight_type = config.down_type;
    const a8::DownBindings down_bindings{
        bindings.output, config.down, bindings.routes, slice(layout.down_codes_offset, layout.down_codes_bytes),
        slice(layout.down_deltas_offset, layout.down_deltas_bytes), slice(layout.down_sums_offset, layout.down_sums_bytes),
        slice(layout.rawdots_offset, layout.rawdots_bytes), bindings.status, {}};
    // all admission is complete before the first enqueue (src/hip_moe_experts_launcher.hip:1440-1441,1472-1473)
    a8::validate(request, bindings);
    a8::validate_down(down_request, down_bindings);

    float* accumulation = reinterpret_cast<float*>(temporary.address + layout.accumulation_offset);
    a8::SlotMergeTail tail;
    tail.tickets = reinterpret_cast<std::uint32_t*>(temporary.address + layout.ticket_offset);     // not used by this library's tail
    tail.route_weights = reinterpret_cast<const float*>(route_weights.address);
    tail.accumulation = accumulation;
    tail.output = reinterpret_cast<void*>(output.address);
    tail.output_bf16 = config.bf16_activation;
    tail.bf16_commit = config.bf16_activation;
    tail.record = config.first_error_record;
    tail.domain = 2;                                                                                // DeferredMoeDomain::q4k_a8

    // the fused prologue clears the accumulation (the status word that follows it is overwritten by the same workgroup),
    // checks routes and route weights, quantises and projects (:1511-1514); then h and its A8 image; then the down rows with
    // the ordered merge, the commit test and the first-error record in their tail
    a8::enqueue_serial_prologue_probe(request, bindings, accumulation, static_cast<unsigned>(layout.accumulation_bytes / 4U),
                                      tail.route_weights, config.stream);
    a8::enqueue_down_activation_quantize(down_request, down_bindings, config.stream);
    a8::enqueue_down_rawdots(down_request, down_bindings, tail, config.stream);
}

// The entry of the dispatch table (ExecutionLauncher, include/strix/launch_dispatch.hpp:19-26): the key names the runtime step, the
// implementation identity hashes the two arithmetic tokens this library declares for the layer's tensor types.
inline ::strix::ExecutionLauncher moe_experts_launcher(MoeExpertsLauncherConfig& config) {
    ::strix::ExecutionLauncher launcher;
    launcher.key = "moe_experts.mi355.a8";
    launcher.implementation_identity = detail::fnv1a(moe_q4k_a8::down_numerical_identity(config.down_type),
                                                     detail::fnv1a(moe_q4k_a8::numerical_identity_for_gate_type(config.gate_type)));
    launcher.function = &launch_moe_experts;
    launcher.user_data = &config;
    return launcher;
}

inline void register_moe_experts(::strix::ExecutionLauncherRegistry& registry, MoeExpertsLauncherConfig& config) {
    registry.add_runtime_launcher(::strix::SerialOp::moe_experts, moe_experts_launcher(config));
}

}  // namespace strix::mi355

// the signature the dispatch table asks for
static_assert(std::is_same_v<decltype(&strix::mi355::launch_moe_experts), strix::ExecutionLaunchFunction>);
