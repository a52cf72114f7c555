// The HIP binding of the registry's runtime callbacks for this library: what the reference's HIP backend installs with
// bind_native_runtime (src/hip/weight/runtime.hpp:4-10, src/hip/weight/runtime.cpp:17-47 over src/weight/native_runtime.hpp:71-125),
// with this library's typed launcher as the enqueue callback. Same callback meanings and error mapping (out of memory ->
// memory_budget, any other HIP failure -> device_failure with the runtime's message), host C++ over the HIP runtime API only.
// Differences, all on the host side:
//   * convert copies the view's payload as it is (host or device memory, one asynchronous copy on the context's stream followed
//     by a wait for it); the reference reads a file-backed source in 64 KB chunks through its own reader;
//   * retirement is collected on the caller's threads (at every retire call and at shutdown_native_runtime), not by a
//     service thread: an allocation is freed once all its events have completed and its unresolved streams are idle, a failed
//     free is kept (never retried), and shutdown drains what is left.
#pragma once
#include <hip/hip_runtime_api.h>

#include <mutex>
#include <utility>

#include "strix_mi355.hpp"

namespace strix::mi355::weight {
namespace detail {
inline Status hip_status(hipError_t error) {
    if (error == hipSuccess) return {Error::ok, {}};
    return {error == hipErrorOutOfMemory ? Error::memory_budget : Error::device_failure, hipGetErrorString(error)};
}
struct Pending { void* data; Retirement retirement; std::uint32_t device; bool quarantined = false; };
struct RetirementList {
    std::mutex mutex;
    std::vector<Pending> pending;
    std::size_t reclaimed = 0;
    void collect_locked(bool drain) {
        for (auto it = pending.begin(); it != pending.end();) {
            if (it->quarantined) { ++it; continue; }
            bool done = hipSetDevice(static_cast<int>(it->device)) == hipSuccess;
            for (void* stream : it->retirement.unresolved_streams) {
                if (!done) break;
                done = (drain ? hipStreamSynchronize(static_cast<hipStream_t>(stream)) : hipStreamQuery(static_cast<hipStream_t>(stream))) == hipSuccess;
            }
            for (void* event : it->retirement.events) {
                if (!done) break;
                done = (drain ? hipEventSynchronize(static_cast<hipEvent_t>(event)) : hipEventQuery(static_cast<hipEvent_t>(event))) == hipSuccess;
            }
            if (!done) { ++it; continue; }
            if (hipFree(it->data) != hipSuccess) { it->quarantined = true; ++it; continue; }       // uncertain ownership: never retried
            for (void* event : it->retirement.events) (void)hipEventDestroy(static_cast<hipEvent_t>(event));
            it = pending.erase(it);                                                                // (releases the reservation)
            ++reclaimed;
        }
    }
    void retire(Pending item) {
        std::lock_guard<std::mutex> lock(mutex);
        pending.push_back(std::move(item));
        collect_locked(false);
    }
};
inline RetirementList& retirements() { static RetirementList list; return list; }
}  // namespace detail

// allocations retired and not yet reclaimed / reclaimed so far (for tests and for a cache's accounting)
inline std::size_t retirements_pending() { auto& l = detail::retirements(); std::lock_guard<std::mutex> lock(l.mutex); l.collect_locked(false); return l.pending.size(); }
inline std::size_t retirements_reclaimed() { auto& l = detail::retirements(); std::lock_guard<std::mutex> lock(l.mutex); return l.reclaimed; }
// Terminal: call after all contexts stopped submitting work (src/hip/weight/runtime.hpp:9-10).
inline void shutdown_native_runtime() { auto& l = detail::retirements(); std::lock_guard<std::mutex> lock(l.mutex); l.collect_locked(true); }

inline Status bind_native_runtime(void* stream, std::uint32_t device, ExecutionContext& context, Hardware& hardware) {
    using detail::hip_status;
    if (device > static_cast<std::uint32_t>(INT32_MAX)) return {Error::device_failure, "device index overflow"};
    Status status = hip_status(hipSetDevice(static_cast<int>(device)));
    if (!status) return status;
    hipDeviceProp_t properties{};
    status = hip_status(hipGetDeviceProperties(&properties, static_cast<int>(device)));
    if (!status) return status;
    std::size_t free_bytes = 0, total_bytes = 0;
    status = hip_status(hipMemGetInfo(&free_bytes, &total_bytes));
    if (!status) return status;
    Hardware h{};
    h.backend = Backend::hip;
    h.arch = properties.gcnArchName;
    h.compiler_id = current_compiler_id();
    h.device_class = h.arch;
    h.free_bytes = free_bytes;
    h.warp_or_wave = static_cast<std::uint32_t>(properties.warpSize);
    h.shared_bytes_per_sm = static_cast<std::uint32_t>(properties.sharedMemPerMultiprocessor);
    // (rates and the image budget come from deployment, as in the reference: nothing is guessed here)
    auto callbacks = std::make_shared<RuntimeCallbacks>();
    callbacks->allocate = [device](std::uint64_t bytes, void*& data) -> Status {
        Status s = hip_status(hipSetDevice(static_cast<int>(device)));
        if (!s) return s;
        if (bytes > SIZE_MAX) return {Error::memory_budget, "allocation size overflow"};
        return hip_status(hipMalloc(&data, static_cast<std::size_t>(bytes ? bytes : 1)));
    };
    callbacks->free = [device](void* data) { if (hipSetDevice(static_cast<int>(device)) == hipSuccess) (void)hipFree(data); };
    callbacks->record_event = [device](ExecutionContext& c, void*& value) -> Status {
        Status s = hip_status(hipSetDevice(static_cast<int>(device)));
        if (!s) return s;
        hipEvent_t event{};
        s = hip_status(hipEventCreateWithFlags(&event, hipEventDisableTiming));
        if (!s) return s;
        s = hip_status(hipEventRecord(event, static_cast<hipStream_t>(c.stream)));
        if (!s) { (void)hipEventDestroy(event); return s; }
        value = event;
        return s;
    };
    callbacks->wait_event = [device](ExecutionContext& c, void* event) -> Status {
        Status s = hip_status(hipSetDevice(static_cast<int>(device)));
        if (!s) return s;
        return hip_status(hipStreamWaitEvent(static_cast<hipStream_t>(c.stream), static_cast<hipEvent_t>(event), 0));
    };
    callbacks->event_complete = [device](void* event) { return hipSetDevice(static_cast<int>(device)) == hipSuccess && hipEventQuery(static_cast<hipEvent_t>(event)) == hipSuccess; };
    callbacks->destroy_event = [device](void* event) { if (hipSetDevice(static_cast<int>(device)) == hipSuccess) (void)hipEventDestroy(static_cast<hipEvent_t>(event)); };
    callbacks->convert = [device](const WeightView& w, const Plan& p, void* data, ExecutionContext& c) -> Status {
        if (p.selected.strategy != Strategy::native) return {Error::unsupported_arithmetic, "image conversion source not registered"};
        if (!w.payload || !data) return {Error::malformed, "image conversion without a payload or a destination"};
        Status s = hip_status(hipSetDevice(static_cast<int>(device)));
        if (!s) return s;
        s = hip_status(hipMemcpyAsync(data, w.payload, static_cast<std::size_t>(w.payload_bytes), hipMemcpyDefault, static_cast<hipStream_t>(c.stream)));
        const Status copied = hip_status(hipStreamSynchronize(static_cast<hipStream_t>(c.stream)));      // the image is ready before any consumer is told so
        if (!s) return s;
        return copied;
    };
    callbacks->retire = [device](void* data, Retirement retirement, ExecutionContext) {
        detail::retirements().retire({data, std::move(retirement), device});
    };
    callbacks->enqueue = [](const Plan& plan, const WeightView& weight, const KernelArguments& args, void* output, void* workspace, std::size_t bytes, ExecutionContext& c) -> Status {
        // the typed launch runs on the context's stream: the envelope's own stream field is overridden
        if (args.schema == q8_tree32_kernel && args.bytes == sizeof(DenseArguments) && args.data) {
            DenseArguments launch = *static_cast<const DenseArguments*>(args.data);
            launch.stream.stream = c.stream;
            KernelArguments bound = args;
            bound.data = &launch;
            return enqueue(plan, weight, bound, output, workspace, bytes);
        }
        return enqueue(plan, weight, args, output, workspace, bytes);
    };
    context = {Backend::hip, stream, device, std::move(callbacks)};
    hardware = std::move(h);
    return {Error::ok, {}};
}
}  // namespace strix::mi355::weight
