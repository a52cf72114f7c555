// Calls the library on the GPU through the C++ mirror of the reference's interfaces (strix_mi355.hpp) and checks the bits
// against the CPU oracle (liboracle.so, the checker). Built by __graft_entry__.build() with hipcc as host C++; run as a child
// process by tests/test_gpu_cpp_mirror.py. Exit status = number of failed checks.
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "strix_mi355.hpp"
#include "strix_mi355_runtime.hpp"
extern "C" {
#include "strix_oracle.h"
}

namespace m = strix::mi355;

static int failures = 0;
static void expect(bool ok, const char* what) {
    std::printf("%s %s\n", ok ? "PASS" : "FAIL", what);
    std::fflush(stdout);
    if (!ok) ++failures;
}
static void hip(hipError_t e, const char* what) {
    if (e != hipSuccess) { std::printf("HIP error in %s: %s\n", what, hipGetErrorString(e)); std::exit(100); }
}
template <class T> struct Dev {                        // a device array with its host copy
    T* p = nullptr;
    size_t n = 0;
    explicit Dev(size_t count) : n(count) { hip(hipMalloc(reinterpret_cast<void**>(&p), (count ? count : 1) * sizeof(T)), "hipMalloc"); hip(hipMemset(p, 0, (count ? count : 1) * sizeof(T)), "hipMemset"); }
    explicit Dev(const std::vector<T>& h) : Dev(h.size()) { put(h); }
    ~Dev() { (void)hipFree(p); }
    Dev(const Dev&) = delete;
    void put(const std::vector<T>& h) { hip(hipMemcpy(p, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice), "H2D"); }
    std::vector<T> get() const { std::vector<T> h(n); hip(hipMemcpy(h.data(), p, n * sizeof(T), hipMemcpyDeviceToHost), "D2H"); return h; }
    m::moe_q4k_a8::DeviceBytes bytes() const { return {reinterpret_cast<std::uintptr_t>(p), static_cast<std::uint64_t>(n * sizeof(T))}; }
};
template <class T> static bool same_bits(const std::vector<T>& a, const std::vector<T>& b) {
    return a.size() == b.size() && std::memcmp(a.data(), b.data(), a.size() * sizeof(T)) == 0;
}
static std::uint16_t bf16_rne(float f) {
    std::uint32_t b; std::memcpy(&b, &f, 4);
    return static_cast<std::uint16_t>((b + 0x7fffU + ((b >> 16) & 1U)) >> 16);
}
static float bf16_value(std::uint16_t h) { const std::uint32_t b = static_cast<std::uint32_t>(h) << 16; float f; std::memcpy(&f, &b, 4); return f; }

constexpr std::uint32_t H = 512, I = 256, E = 4, K = 2, T = 3;
static std::mt19937 rng(12345);
static std::vector<float> normal(size_t n, float scale) {
    std::normal_distribution<float> d(0.0F, scale);
    std::vector<float> v(n);
    for (auto& x : v) x = d(rng);
    return v;
}
static std::vector<std::uint8_t> q4k_tensor(size_t rows, std::uint32_t width, float scale) {
    std::vector<std::uint8_t> out(rows * (width / 256) * 144);
    const std::vector<float> w = normal(rows * width, scale);
    for (size_t r = 0; r < rows; ++r) orc_quantize_q4_k_row(w.data() + r * width, width, out.data() + r * (width / 256) * 144);
    return out;
}
static std::vector<std::uint8_t> q8_0_tensor(size_t rows, std::uint32_t width, float scale) {
    std::vector<std::uint8_t> out(rows * (width / 32) * 34);
    const std::vector<float> w = normal(rows * width, scale);
    for (size_t r = 0; r < rows; ++r) orc_quantize_q8_0_row(w.data() + r * width, width, out.data() + r * (width / 32) * 34);
    return out;
}

// ----------------------------------------------------------------------------------------------- the dense kernel table
static void kernel_table() {
    const m::cpu::Kernels& k = m::cpu::mi355_kernels();
    const std::uint32_t width = 1024, count = 96;
    const std::vector<float> x = normal(width, 1.0F);
    Dev<float> dx(x), dd(width / 32), dy(width), dout(count);
    Dev<std::int8_t> dc(width);
    Dev<std::int32_t> ds(width / 32);
    k.quantize_a8(dx.p, width, dc.p, dd.p, ds.p);
    std::vector<std::int8_t> c(width); std::vector<float> d(width / 32); std::vector<std::int32_t> s(width / 32);
    orc_quantize_a8(x.data(), width, c.data(), d.data(), s.data(), 1);
    expect(same_bits(dc.get(), c) && same_bits(dd.get(), d) && same_bits(ds.get(), s), "Kernels::quantize_a8 == oracle");
    const std::vector<std::uint8_t> w = q8_0_tensor(count, width, 0.05F);
    Dev<std::uint8_t> dw(w);
    const m::cpu::Q8a8View view{dw.p, dc.p, dd.p, dout.p, width / 32 * 34, width, count, 1, width, count, 0};
    k.gemv_q8_0_a8(view, m::cpu::Stream{});
    std::vector<float> want(count);
    const orc_q8a8_view ov{w.data(), c.data(), d.data(), want.data(), width / 32 * 34, width, count, 1, width, count, 0};
    orc_gemv_q8_0_a8(&ov, 1);
    expect(same_bits(dout.get(), want), "Kernels::gemv_q8_0_a8 == oracle");
    const std::vector<float> g = normal(width, 1.0F);
    Dev<float> dg(g);
    k.rmsnorm_f32(dx.p, dg.p, width, 1e-6F, dy.p, 1, m::cpu::Stream{});
    std::vector<float> yn(width);
    orc_rmsnorm_f32(x.data(), g.data(), width, 1e-6F, yn.data(), 1);
    expect(same_bits(dy.get(), yn), "Kernels::rmsnorm_f32 == oracle");
    bool threw = false;
    try { k.quantize_a8(dx.p, 33, dc.p, dd.p, ds.p); } catch (const std::invalid_argument&) { threw = true; }
    expect(threw, "Kernels::quantize_a8 throws std::invalid_argument for width % 32 != 0");

    // the same product through the typed registry envelope
    namespace wt = m::weight;
    Dev<float> dout2(count);
    const wt::WeightView weight{7, {"gguf.q8_0", 1}, wt::Shape{{width, count, 0, 0}, 2}, dw.p, w.size()};
    wt::DenseArguments args{view, m::cpu::Stream{}};
    args.view.out = dout2.p;
    expect(static_cast<bool>(wt::enqueue_dense(weight, args)) && same_bits(dout2.get(), want), "weight::enqueue_dense (typed envelope) == oracle");
    std::size_t n = 0;
    wt::Plan plan{wt::candidates(n)[0]};
    wt::KernelArguments envelope = wt::arguments(args);
    envelope.abi_revision = 1;
    expect(wt::enqueue(plan, weight, envelope, dout2.p, nullptr, 0).code == wt::Error::malformed, "weight::enqueue refuses an envelope of another ABI revision: malformed");
    envelope = wt::arguments(args);
    plan.selected.arithmetic = wt::ArithmeticId{"cpu-q8a8-tree32", 2};
    expect(wt::enqueue(plan, weight, envelope, dout2.p, nullptr, 0).code == wt::Error::unsupported_arithmetic, "weight::enqueue refuses another arithmetic: unsupported_arithmetic");
    plan = wt::Plan{wt::candidates(n)[0]};
    wt::DenseArguments bad = args;
    bad.view.x_stride = width + 8;
    envelope = wt::arguments(bad);
    expect(wt::enqueue(plan, weight, envelope, dout2.p, nullptr, 0).code == wt::Error::unsupported_shape, "weight::enqueue refuses a stride that is no multiple of 32: unsupported_shape");
    wt::WeightView other = weight;
    other.shape.dims[1] = count + 1;
    envelope = wt::arguments(args);
    expect(wt::enqueue(plan, other, envelope, dout2.p, nullptr, 0).code == wt::Error::unsupported_shape, "weight::enqueue refuses a weight whose shape differs from the launch");
}

// ----------------------------------------------------------------------------------------------- the registry's runtime callbacks
// include/strix/weight/cache.hpp:14-33 bound to HIP and to this library: a weight image allocated, uploaded from host memory
// and launched through the context, on a stream of its own, with its last use recorded and the allocation retired.
static void weight_runtime() {
    namespace wt = m::weight;
    hipStream_t stream{};
    hip(hipStreamCreate(&stream), "hipStreamCreate");
    wt::ExecutionContext context;
    wt::Hardware hardware{};
    expect(static_cast<bool>(wt::bind_native_runtime(stream, 0, context, hardware)) && context.backend == wt::Backend::hip && context.stream == stream &&
               context.callbacks && hardware.backend == wt::Backend::hip && hardware.arch.rfind("gfx950", 0) == 0 && hardware.warp_or_wave == 64 &&
               hardware.free_bytes > 0 && !hardware.compiler_id.empty(),
           "weight::bind_native_runtime: HIP context on the caller's stream, hardware gfx950 / wave 64");
    wt::RuntimeAdapter none;
    wt::ExecutionContext unbound;
    expect(wt::bind_runtime(wt::Backend::hip, none, stream, 0, unbound, hardware).code == wt::Error::unsupported_backend, "weight::bind_runtime refuses an adapter without callbacks");
    wt::RuntimeAdapter adapter{context.callbacks, [](std::uint32_t, wt::Hardware& h) { h.backend = wt::Backend::cpu; return wt::Status{wt::Error::ok, {}}; }};
    expect(wt::bind_runtime(wt::Backend::hip, adapter, stream, 0, unbound, hardware).code == wt::Error::unsupported_backend, "weight::bind_runtime refuses a capability query of another backend");
    adapter.query_hardware = [](std::uint32_t, wt::Hardware& h) { h.backend = wt::Backend::hip; h.arch = "gfx950"; return wt::Status{wt::Error::ok, {}}; };
    expect(static_cast<bool>(wt::bind_runtime(wt::Backend::hip, adapter, stream, 0, unbound, hardware)) && unbound.callbacks == context.callbacks, "weight::bind_runtime installs the adapter's callbacks");

    const std::uint32_t width = 2048, count = 160;
    const std::vector<float> x = normal(width, 1.0F);
    std::vector<std::int8_t> c(width); std::vector<float> d(width / 32); std::vector<std::int32_t> sums(width / 32);
    orc_quantize_a8(x.data(), width, c.data(), d.data(), sums.data(), 1);
    const std::vector<std::uint8_t> w = q8_0_tensor(count, width, 0.05F);
    std::vector<float> want(count);
    const orc_q8a8_view ov{w.data(), c.data(), d.data(), want.data(), width / 32 * 34, width, count, 1, width, count, 0};
    orc_gemv_q8_0_a8(&ov, 1);
    Dev<std::int8_t> dc(c);
    Dev<float> dd(d), dout(count);

    // the image: allocate, upload from HOST memory, then the typed launch on the context's stream
    void* image = nullptr;
    const wt::WeightView host_view{11, {"gguf.q8_0", 1}, wt::Shape{{width, count, 0, 0}, 2}, w.data(), w.size()};
    std::size_t n = 0;
    wt::Plan plan{wt::candidates(n)[0]};
    bool ok = static_cast<bool>(context.callbacks->allocate(w.size(), image)) && image != nullptr;
    ok = ok && static_cast<bool>(context.callbacks->convert(host_view, plan, image, context));
    wt::WeightView device_view = host_view;
    device_view.payload = static_cast<const std::uint8_t*>(image);
    wt::DenseArguments args{m::cpu::Q8a8View{device_view.payload, dc.p, dd.p, dout.p, width / 32 * 34, width, count, 1, width, count, 0}, m::cpu::Stream{}};
    ok = ok && static_cast<bool>(wt::enqueue(plan, device_view, wt::arguments(args), dout.p, nullptr, 0, context));
    void* last_use = nullptr;
    ok = ok && static_cast<bool>(context.callbacks->record_event(context, last_use)) && last_use != nullptr;
    wt::ExecutionContext other = context;
    other.stream = nullptr;                                             // a consumer on another stream waits for the producer's event
    ok = ok && static_cast<bool>(context.callbacks->wait_event(other, last_use));
    hip(hipStreamSynchronize(stream), "hipStreamSynchronize");
    expect(ok && context.callbacks->event_complete(last_use) && same_bits(dout.get(), want), "weight runtime: allocate + convert + enqueue on the context's stream == oracle");

    // the refusals of the launch through a context, in the reference's order
    wt::ExecutionContext cpu_context = context;
    cpu_context.backend = wt::Backend::cpu;
    wt::KernelArguments envelope = wt::arguments(args);
    expect(wt::enqueue(plan, device_view, envelope, dout.p, nullptr, 0, cpu_context).code == wt::Error::unsupported_backend, "weight::enqueue(context) refuses another backend");
    wt::WeightView q4 = device_view;
    q4.storage = wt::FormatId{"gguf.q4_k", 1};
    expect(wt::enqueue(plan, q4, envelope, dout.p, nullptr, 0, context).code == wt::Error::unknown_format, "weight::enqueue(context) refuses another storage");
    wt::Plan hungry = plan;
    hungry.workspace_bytes = 64;
    expect(wt::enqueue(hungry, device_view, envelope, dout.p, nullptr, 0, context).code == wt::Error::memory_budget, "weight::enqueue(context) refuses a missing workspace");
    expect(wt::enqueue(plan, device_view, envelope, nullptr, nullptr, 0, context).code == wt::Error::malformed, "weight::enqueue(context) refuses a null output");
    wt::ExecutionContext bare{wt::Backend::hip, stream, 0, nullptr};
    expect(wt::enqueue(plan, device_view, envelope, dout.p, nullptr, 0, bare).code == wt::Error::unsupported_arithmetic, "weight::enqueue(context) refuses a context without a launcher");
    wt::Plan staged = plan;
    staged.selected.strategy = wt::Strategy::converted;
    expect(context.callbacks->convert(host_view, staged, image, context).code == wt::Error::unsupported_arithmetic, "weight runtime: convert refuses a strategy without a registered source");

    // retirement: the allocation, its last-use event and its budget token go together; reclaimed once the event has completed
    auto token = std::make_shared<int>(1);
    std::weak_ptr<int> watch = token;
    const std::size_t before = wt::retirements_reclaimed();
    wt::Retirement retirement;
    retirement.events.push_back(last_use);
    retirement.reservation = std::move(token);
    context.callbacks->retire(image, std::move(retirement), context);
    wt::shutdown_native_runtime();
    expect(wt::retirements_pending() == 0 && wt::retirements_reclaimed() == before + 1 && watch.expired(), "weight runtime: a retired image is reclaimed after its last use, its reservation released");
    hip(hipStreamDestroy(stream), "hipStreamDestroy");
}

// ----------------------------------------------------------------------------------------------- one expert layer, three ways
struct Layer {
    std::vector<std::uint8_t> gate = q4k_tensor(size_t(E) * I, H, 0.05F), up = q4k_tensor(size_t(E) * I, H, 0.05F);
    std::vector<std::uint8_t> down = q4k_tensor(size_t(E) * H, I, 0.05F), down8 = q8_0_tensor(size_t(E) * H, I, 0.05F);
    std::vector<std::uint16_t> x;                          // bf16 rows
    std::vector<float> x32;
    std::vector<std::uint32_t> routes{1, 3, 0, 2, 3, 1};   // [T][K]
    std::vector<float> weights{0.75F, 0.25F, 0.5F, 0.5F, 0.125F, 0.875F};
    std::vector<std::int8_t> c; std::vector<float> d; std::vector<std::int32_t> s;
    Layer() : c(T * H), d(T * H / 32), s(T * H / 32) {
        const std::vector<float> raw = normal(T * H, 1.0F);
        for (float v : raw) { x.push_back(bf16_rne(v)); x32.push_back(bf16_value(x.back())); }
        for (std::uint32_t t = 0; t < T; ++t) orc_quantize_a8(x32.data() + t * H, H, c.data() + t * H, d.data() + t * (H / 32), s.data() + t * (H / 32), 0);
    }
    // the oracle's whole job with the given down tensor
    struct Result { std::vector<float> gate, up, h, rawdots; std::vector<std::int8_t> hc; std::vector<float> hd; std::vector<std::int32_t> hs; };
    Result oracle(const std::vector<std::uint8_t>& down_tensor, std::uint32_t down_type) const {
        Result r;
        const size_t n = size_t(T) * K;
        r.gate.resize(n * I); r.up.resize(n * I); r.h.resize(n * I); r.rawdots.resize(n * H); r.hc.resize(n * I); r.hd.resize(n * I / 32); r.hs.resize(n * I / 32);
        std::vector<std::uint32_t> status(T);
        const std::uint64_t grb = H / 256 * 144, drb = down_type == 12 ? I / 256 * 144 : I / 32 * 34;
        const orc_expert_weights w{H, I, E, K, 12, down_type, gate.data(), up.data(), down_tensor.data(), grb * I, grb, drb * H, drb, 0, INFINITY};
        const orc_expert_job job{c.data(), d.data(), s.data(), routes.data(), T, r.gate.data(), r.up.data(), r.h.data(), r.hc.data(), r.hd.data(), r.hs.data(),
                                 r.rawdots.data(), status.data()};
        orc_routed_experts(&w, &job, 1);
        return r;
    }
};

static void a8_single_row(const Layer& L) {
    namespace a8 = m::moe_q4k_a8;
    const Layer::Result ref = L.oracle(L.down, 12);
    Dev<std::uint8_t> gate(L.gate), up(L.up), down(L.down);
    Dev<std::uint16_t> input(std::vector<std::uint16_t>(L.x.begin(), L.x.begin() + H));
    Dev<std::uint32_t> routes(std::vector<std::uint32_t>(L.routes.begin(), L.routes.begin() + K)), status(1), aggregate(1), record(2);
    Dev<std::int8_t> codes(H), hcodes(K * I);
    Dev<float> deltas(H / 32), output(K * 2 * I), hdeltas(K * I / 32), rawdots(K * H), acc(H), route_w(std::vector<float>(L.weights.begin(), L.weights.begin() + K));
    Dev<std::int32_t> sums(H / 32), hsums(K * I / 32);
    Dev<std::uint16_t> y(H);
    a8::Request q;
    q.enabled = true; q.approved_numerical_identity = a8::numerical_identity_for_gate_type(12); q.input = a8::InputKind::bf16;
    q.shape = a8::Shape{H, I, E, K, 1};
    const a8::Bindings b{input.bytes(), gate.bytes(), up.bytes(), routes.bytes(), codes.bytes(), deltas.bytes(), sums.bytes(), status.bytes(), output.bytes()};
    a8::validate(q, b);
    a8::enqueue_probe(q, b, nullptr);
    const std::vector<float> out = output.get();
    bool ok = true;
    for (std::uint32_t k = 0; k < K; ++k)
        ok = ok && std::memcmp(out.data() + (k * 2) * I, ref.gate.data() + k * I, I * 4) == 0 && std::memcmp(out.data() + (k * 2 + 1) * I, ref.up.data() + k * I, I * 4) == 0;
    expect(ok, "moe_q4k_a8::enqueue_probe: output[(slot * 2 + which) * rows + i] == oracle gate / up rows");
    a8::DownRequest dq;
    dq.enabled = true; dq.approved_numerical_identity = a8::down_numerical_identity(12); dq.shape = a8::DownShape{H, I, E, K}; dq.weight_type = 12;
    const a8::DownBindings db{output.bytes(), down.bytes(), routes.bytes(), hcodes.bytes(), hdeltas.bytes(), hsums.bytes(), rawdots.bytes(), status.bytes(), aggregate.bytes()};
    a8::validate_down(dq, db);
    a8::enqueue_down_activation_quantize(dq, db, nullptr);
    expect(same_bits(hcodes.get(), std::vector<std::int8_t>(ref.hc.begin(), ref.hc.begin() + K * I)) &&
           same_bits(hdeltas.get(), std::vector<float>(ref.hd.begin(), ref.hd.begin() + K * I / 32)), "moe_q4k_a8::enqueue_down_activation_quantize == oracle h image");
    a8::SlotMergeTail tail;
    tail.route_weights = route_w.p; tail.accumulation = acc.p; tail.output = y.p; tail.output_bf16 = true; tail.bf16_commit = true; tail.record = record.p; tail.domain = 2;
    a8::enqueue_down_rawdots(dq, db, tail, nullptr);
    expect(same_bits(rawdots.get(), std::vector<float>(ref.rawdots.begin(), ref.rawdots.begin() + K * H)), "moe_q4k_a8::enqueue_down_rawdots (merge tail) rawdots == oracle");
    std::vector<float> want(H);
    orc_combine(0, 1, K, H, L.weights.data(), L.routes.data(), ref.rawdots.data(), nullptr, want.data());
    std::vector<std::uint16_t> want16;
    for (float v : want) want16.push_back(bf16_rne(v));
    expect(same_bits(acc.get(), want) && same_bits(y.get(), want16) && status.get()[0] == 0 && record.get()[0] == 0, "slot merge tail: accumulation, bf16 output, clean status");
    bool threw = false;
    q.approved_numerical_identity = "not the approved arithmetic";
    try { a8::enqueue_probe(q, b, nullptr); } catch (const std::invalid_argument&) { threw = true; }
    expect(threw, "moe_q4k_a8::enqueue_probe throws std::invalid_argument without the identity approval");
}

// The serial row's fused prologue, the quantiser alone, and the alignment rule of the down weights.
static void a8_serial_forms(const Layer& L) {
    namespace a8 = m::moe_q4k_a8;
    const Layer::Result ref = L.oracle(L.down, 12);
    Dev<std::uint8_t> gate(L.gate), up(L.up);
    Dev<std::uint16_t> input(std::vector<std::uint16_t>(L.x.begin(), L.x.begin() + H));
    Dev<std::uint32_t> routes(std::vector<std::uint32_t>(L.routes.begin(), L.routes.begin() + K)), status(std::vector<std::uint32_t>{0xabcdU});
    Dev<std::int8_t> codes(H);
    Dev<float> deltas(H / 32), output(K * 2 * I), clear(std::vector<float>(H + 3, 5.0F)), route_w(std::vector<float>(L.weights.begin(), L.weights.begin() + K));
    Dev<std::int32_t> sums(H / 32);
    a8::Request q;
    q.enabled = true; q.approved_numerical_identity = a8::numerical_identity_for_gate_type(12); q.input = a8::InputKind::bf16;
    q.shape = a8::Shape{H, I, E, K, 1};
    const a8::Bindings b{input.bytes(), gate.bytes(), up.bytes(), routes.bytes(), codes.bytes(), deltas.bytes(), sums.bytes(), status.bytes(), output.bytes()};
    a8::enqueue_serial_prologue_probe(q, b, clear.p, H, route_w.p, nullptr);
    const std::vector<float> out = output.get(), cleared = clear.get();
    bool ok = status.get()[0] == 0;                                       // the stale word is overwritten
    for (std::uint32_t i = 0; i < H + 3; ++i) ok = ok && cleared[i] == (i < H ? 0.0F : 5.0F);
    ok = ok && same_bits(codes.get(), std::vector<std::int8_t>(L.c.begin(), L.c.begin() + H)) && same_bits(deltas.get(), std::vector<float>(L.d.begin(), L.d.begin() + H / 32));
    for (std::uint32_t k = 0; k < K; ++k)
        ok = ok && std::memcmp(out.data() + (k * 2) * I, ref.gate.data() + k * I, I * 4) == 0 && std::memcmp(out.data() + (k * 2 + 1) * I, ref.up.data() + k * I, I * 4) == 0;
    expect(ok, "moe_q4k_a8::enqueue_serial_prologue_probe: cleared words, overwritten status, image and gate / up rows == oracle");
    // a non-finite route weight: bit 1, nothing stored
    Dev<float> bad_w(std::vector<float>{0.5F, INFINITY});
    Dev<std::int8_t> codes2(std::vector<std::int8_t>(H, 77));
    Dev<float> output2(std::vector<float>(K * 2 * I, -7.0F));
    const a8::Bindings b2{input.bytes(), gate.bytes(), up.bytes(), routes.bytes(), codes2.bytes(), deltas.bytes(), sums.bytes(), status.bytes(), output2.bytes()};
    a8::enqueue_serial_prologue_probe(q, b2, clear.p, H, bad_w.p, nullptr);
    expect(status.get()[0] == a8::invalid_route && codes2.get() == std::vector<std::int8_t>(H, 77) && output2.get() == std::vector<float>(K * 2 * I, -7.0F),
           "moe_q4k_a8::enqueue_serial_prologue_probe: a non-finite route weight sets bit 1 and stores neither image nor rows");
    Dev<std::uint32_t> status3(1);
    const a8::Bindings b3{input.bytes(), gate.bytes(), up.bytes(), routes.bytes(), codes2.bytes(), deltas.bytes(), sums.bytes(), status3.bytes(), output2.bytes()};
    a8::enqueue_quantize_only(q, b3, nullptr);
    expect(status3.get()[0] == 0 && same_bits(codes2.get(), std::vector<std::int8_t>(L.c.begin(), L.c.begin() + H)) && output2.get() == std::vector<float>(K * 2 * I, -7.0F),
           "moe_q4k_a8::enqueue_quantize_only: the image == oracle, no projection");
    // the down weights: this library asks 16 bytes of every class; a Q8_0 tensor on 2 bytes, which the reference admits
    // (src/moe_a8_down_contract.cpp:72-73), is refused by name
    Dev<std::uint8_t> down8(std::vector<std::uint8_t>(L.down8.size() + 16));
    Dev<std::int8_t> hcodes(K * I);
    Dev<float> hdeltas(K * I / 32), rawdots(K * H);
    Dev<std::int32_t> hsums(K * I / 32);
    Dev<std::uint32_t> dstatus(1), aggregate(1);
    a8::DownRequest dq;
    dq.enabled = true; dq.approved_numerical_identity = a8::down_numerical_identity(8); dq.shape = a8::DownShape{H, I, E, K}; dq.weight_type = 8;
    a8::DownBindings db{output.bytes(), a8::DeviceBytes{reinterpret_cast<std::uintptr_t>(down8.p), L.down8.size()}, routes.bytes(), hcodes.bytes(), hdeltas.bytes(),
                        hsums.bytes(), rawdots.bytes(), dstatus.bytes(), aggregate.bytes()};
    bool admitted = true, refused = false;
    try { a8::validate_down(dq, db); } catch (const std::invalid_argument&) { admitted = false; }
    db.weights.address += 2;
    try { a8::validate_down(dq, db); } catch (const std::invalid_argument& e) { refused = std::strstr(e.what(), "alignment") != nullptr; }
    expect(admitted && refused, "moe_q4k_a8::validate_down: a Q8_0 weight tensor on 16 bytes is admitted, on 2 bytes refused with the alignment rule");
}

// moe_core::enqueue_combine in both forms (the reference's two bf16-steps shapes, tests/hip_hy4_routed_tests.hip:205-206).
static void combine_forms() {
    namespace mc = m::moe_core;
    using m::moe::CombineForm;
    constexpr unsigned R = 5;
    const auto bf16_values = [](std::vector<float> v) { for (float& x : v) x = bf16_value(bf16_rne(x)); return v; };
    {
        const std::vector<float> eo = bf16_values(normal(size_t(R) * 16 * 1536, 1.0F)), w = normal(R * 16, 0.3F);
        Dev<float> deo(eo), dw(w), y(R * 1536), y2(R * 1536);
        std::vector<float> want(R * 1536), want2(R * 1536);
        mc::enqueue_combine<CombineForm::bf16_steps, 16, 1536>(dw.p, deo.p, nullptr, y.p, R, nullptr);
        orc_combine(ORC_COMBINE_BF16_STEPS, R, 16, 1536, w.data(), nullptr, eo.data(), nullptr, want.data());
        expect(same_bits(y.get(), want), "moe_core::enqueue_combine<bf16_steps, 16, 1536> (latent merge, no base) == oracle");
        const std::vector<float> raw = normal(size_t(R) * 16 * 1536, 1.0F);
        Dev<float> draw(raw);
        mc::enqueue_combine_rounded_eo<CombineForm::bf16_steps, 16, 1536>(dw.p, draw.p, nullptr, y2.p, R, nullptr);
        orc_combine(ORC_COMBINE_BF16_STEPS_ROUNDED_EO, R, 16, 1536, w.data(), nullptr, raw.data(), nullptr, want2.data());
        expect(same_bits(y2.get(), want2), "moe_core::enqueue_combine_rounded_eo<bf16_steps, 16, 1536> == oracle");
    }
    {
        const std::vector<float> eo = bf16_values(normal(size_t(R) * 3072, 1.0F)), sh = bf16_values(normal(size_t(R) * 3072, 1.0F));
        Dev<float> deo(eo), dsh(sh), y(R * 3072);
        std::vector<float> want(R * 3072);
        mc::enqueue_combine<CombineForm::bf16_steps, 1, 3072>(nullptr, deo.p, dsh.p, y.p, R, nullptr);
        orc_combine(ORC_COMBINE_BF16_STEPS, R, 1, 3072, nullptr, nullptr, eo.data(), sh.data(), want.data());
        expect(same_bits(y.get(), want), "moe_core::enqueue_combine<bf16_steps, 1, 3072> (unit weights, shared add) == oracle");
    }
    {
        const std::vector<float> eo = normal(size_t(R) * 8 * 4096, 1.0F), w = normal(R * 8, 0.3F), sh = normal(size_t(R) * 4096, 1.0F);
        Dev<float> deo(eo), dw(w), dsh(sh), y(R * 4096);
        std::vector<float> want(R * 4096);
        const std::vector<std::uint32_t> ids(R * 8, 0U);
        mc::enqueue_combine<CombineForm::fma_f32, 8, 4096>(dw.p, deo.p, dsh.p, y.p, R, nullptr);
        orc_combine(ORC_COMBINE_FMA_SLOT_ORDER, R, 8, 4096, w.data(), ids.data(), eo.data(), sh.data(), want.data());
        expect(same_bits(y.get(), want), "moe_core::enqueue_combine<fma_f32, 8, 4096> (with the shared base) == oracle");
        bool threw = false;
        try { mc::enqueue_combine<CombineForm::fma_f32, 8, 4096>(dw.p, deo.p, nullptr, y.p, R, nullptr); } catch (const std::invalid_argument&) { threw = true; }
        expect(threw, "moe_core::enqueue_combine<fma_f32> throws std::invalid_argument without the shared base");
    }
}

// The union rows form: three rows, each naming all four experts in its own order, so every entry is held by every row.
static void a8_union_rows(const Layer& L) {
    namespace a8 = m::moe_q4k_a8;
    namespace eu = m::moe::expert_union;
    constexpr std::uint32_t R = T, K4 = 4;
    const std::vector<std::uint32_t> routes{2, 0, 3, 1, 0, 1, 2, 3, 3, 2, 1, 0};
    // the oracle's job over the same routes
    std::vector<float> g(R * K4 * I), u(g.size()), h(g.size()), raw(R * K4 * H), hd(R * K4 * I / 32);
    std::vector<std::int8_t> hc(R * K4 * I);
    std::vector<std::int32_t> hs(R * K4 * I / 32);
    std::vector<std::uint32_t> ostatus(R);
    const std::uint64_t grb = H / 256 * 144, drb = I / 256 * 144;
    const orc_expert_weights w{H, I, E, K4, 12, 12, L.gate.data(), L.up.data(), L.down.data(), grb * I, grb, drb * H, drb, 0, INFINITY};
    const orc_expert_job job{L.c.data(), L.d.data(), L.s.data(), routes.data(), R, g.data(), u.data(), h.data(), hc.data(), hd.data(), hs.data(), raw.data(), ostatus.data()};
    orc_routed_experts(&w, &job, 1);
    Dev<std::uint8_t> gate(L.gate), up(L.up), down(L.down), plan(eu::plan_bytes);
    Dev<std::uint16_t> input(L.x);
    Dev<std::uint32_t> droutes(routes), status(1);
    Dev<std::int8_t> codes(R * H), hcodes(R * K4 * I);
    Dev<float> deltas(R * H / 32), output(R * K4 * 2 * I), hdeltas(R * K4 * I / 32), rawdots(R * K4 * H);
    Dev<std::int32_t> sums(R * H / 32), hsums(R * K4 * I / 32);
    a8::Request q;
    q.enabled = true; q.approved_numerical_identity = a8::numerical_identity_for_gate_type(12); q.input = a8::InputKind::bf16;
    q.shape = a8::Shape{H, I, E, K4, R};
    const a8::Bindings b{input.bytes(), gate.bytes(), up.bytes(), droutes.bytes(), codes.bytes(), deltas.bytes(), sums.bytes(), status.bytes(), output.bytes()};
    a8::validate_union(q, b, plan.bytes());
    a8::enqueue_probe_union(q, b, plan.bytes(), nullptr);
    const std::vector<std::uint8_t> got_plan = plan.get();
    const std::vector<eu::Entry> want_plan = eu::build(routes.data(), routes.size(), R, K4, E);
    eu::Header header;
    std::memcpy(&header, got_plan.data(), sizeof header);
    expect(header.count == want_plan.size() && header.count == E && header.rows == R && header.top_k == K4 &&
           std::memcmp(got_plan.data() + sizeof header, want_plan.data(), want_plan.size() * sizeof(eu::Entry)) == 0,
           "moe_q4k_a8::enqueue_probe_union: device plan == moe::expert_union::build");
    const std::vector<float> out = output.get();
    bool ok = true;
    for (std::uint32_t a = 0; a < R * K4; ++a)
        ok = ok && std::memcmp(out.data() + (a * 2) * I, g.data() + a * I, I * 4) == 0 && std::memcmp(out.data() + (a * 2 + 1) * I, u.data() + a * I, I * 4) == 0;
    expect(ok, "moe_q4k_a8::enqueue_probe_union: gate / up rows of every (row, slot) == oracle");
    a8::DownRequest dq;
    dq.enabled = true; dq.approved_numerical_identity = a8::down_numerical_identity(12); dq.shape = a8::DownShape{H, I, E, K4}; dq.weight_type = 12;
    const a8::DownBindings db{output.bytes(), down.bytes(), droutes.bytes(), hcodes.bytes(), hdeltas.bytes(), hsums.bytes(), rawdots.bytes(), status.bytes(), {0, 0}};
    a8::validate_down_union(dq, db, R, plan.bytes());
    a8::enqueue_down_activation_quantize_union(dq, db, R, plan.bytes(), nullptr);
    a8::enqueue_down_rawdots_union(dq, db, R, plan.bytes(), nullptr);
    expect(same_bits(hcodes.get(), hc) && same_bits(hdeltas.get(), hd) && same_bits(rawdots.get(), raw) && status.get()[0] == 0,
           "moe_q4k_a8::enqueue_down_*_union: h image and raw dots == oracle, clean status");
    bool threw = false;
    try { a8::validate_union(q, b, a8::DeviceBytes{plan.bytes().address, eu::plan_bytes - 4}); } catch (const std::invalid_argument&) { threw = true; }
    expect(threw, "moe_q4k_a8::validate_union throws std::invalid_argument for a plan view of another extent");
}

static void strided_rows(const Layer& L) {
    namespace qm = m::qwen_moe;
    const Layer::Result ref = L.oracle(L.down8, 8);
    Dev<std::uint8_t> gate(L.gate), up(L.up), down(L.down8);
    // one record of bytes per row holding every view (all strides equal, none dense)
    const size_t off_in = 0, off_routes = off_in + 2 * H, off_w = off_routes + 16, off_codes = off_w + 16, off_d = off_codes + H, off_s = off_d + H / 8,
                 off_status = off_s + H / 8, off_inter = off_status + 16, off_acc = off_inter + 8 * K * I, off_hc = off_acc + 4 * H, off_hd = off_hc + K * I,
                 off_hs = off_hd + K * I / 8, off_raw = off_hs + K * I / 8, off_out = off_raw + 4 * K * H, stride = off_out + 2 * H + 64;
    std::vector<std::uint8_t> host(T * stride, 0x5A);
    for (std::uint32_t t = 0; t < T; ++t) {
        std::memcpy(host.data() + t * stride + off_in, L.x.data() + t * H, 2 * H);
        std::memcpy(host.data() + t * stride + off_routes, L.routes.data() + t * K, 4 * K);
        std::memcpy(host.data() + t * stride + off_w, L.weights.data() + t * K, 4 * K);
    }
    Dev<std::uint8_t> block(host);
    Dev<std::uint32_t> plan(mi355_moe_plan_words(E, T, K)), summary(1), record(2);
    qm::Rows r;
    const auto at = [&](size_t off) { return block.p + off; };
    r.input = {reinterpret_cast<const std::uint16_t*>(at(off_in)), stride}; r.routes = {reinterpret_cast<const std::uint32_t*>(at(off_routes)), stride};
    r.route_weights = {reinterpret_cast<const float*>(at(off_w)), stride}; r.codes = {reinterpret_cast<std::int8_t*>(at(off_codes)), stride};
    r.deltas = {reinterpret_cast<float*>(at(off_d)), stride}; r.sums = {reinterpret_cast<std::int32_t*>(at(off_s)), stride};
    r.status = {reinterpret_cast<std::uint32_t*>(at(off_status)), stride}; r.intermediates = {reinterpret_cast<float*>(at(off_inter)), stride};
    r.accumulation = {reinterpret_cast<float*>(at(off_acc)), stride}; r.down_codes = {reinterpret_cast<std::int8_t*>(at(off_hc)), stride};
    r.down_deltas = {reinterpret_cast<float*>(at(off_hd)), stride}; r.down_sums = {reinterpret_cast<std::int32_t*>(at(off_hs)), stride};
    r.rawdots = {reinterpret_cast<float*>(at(off_raw)), stride}; r.output = {reinterpret_cast<std::uint16_t*>(at(off_out)), stride};
    r.csr = qm::Csr{plan.p, summary.p};
    r.geometry = qm::Geometry{H, I, E, K};
    qm::Weights w;
    w.gate_type = qm::type_q4_k; w.gate = gate.p; w.up = up.p; w.down_type = qm::type_q8_0; w.down = down.p;
    qm::enqueue_prologue(r, T, H, nullptr);
    qm::enqueue_csr(r, T, nullptr);
    qm::enqueue_project(r, T, w, nullptr);
    qm::enqueue_down(r, T, w, nullptr);
    qm::enqueue_merge(r, T, nullptr);
    qm::enqueue_commit(r, T, record.p, nullptr);
    const std::vector<std::uint8_t> got = block.get();
    std::vector<float> want(T * H);
    orc_combine(0, T, K, H, L.weights.data(), L.routes.data(), ref.rawdots.data(), nullptr, want.data());
    bool raw_ok = true, out_ok = true, codes_ok = true;
    for (std::uint32_t t = 0; t < T; ++t) {
        raw_ok = raw_ok && std::memcmp(got.data() + t * stride + off_raw, ref.rawdots.data() + size_t(t) * K * H, 4 * K * H) == 0;
        codes_ok = codes_ok && std::memcmp(got.data() + t * stride + off_codes, L.c.data() + t * H, H) == 0 &&
                   std::memcmp(got.data() + t * stride + off_hc, ref.hc.data() + size_t(t) * K * I, K * I) == 0;
        for (std::uint32_t o = 0; o < H; ++o) {
            std::uint16_t v; std::memcpy(&v, got.data() + t * stride + off_out + 2 * o, 2);
            out_ok = out_ok && v == bf16_rne(want[t * H + o]);
        }
    }
    expect(codes_ok, "qwen_moe strided stages: A8 images of the input and of h == oracle");
    expect(raw_ok, "qwen_moe strided stages: rawdots == oracle");
    expect(out_ok && summary.get()[0] == 0 && record.get()[0] == 0, "qwen_moe strided stages: bf16 output == oracle merge, clean job");
}

static void executor_job(const Layer& L) {
    namespace ex = m::expert;
    const Layer::Result ref = L.oracle(L.down8, 8);
    Dev<std::uint8_t> gate(L.gate), up(L.up), down(L.down8);
    Dev<std::int8_t> c(L.c);
    Dev<float> d(L.d);
    Dev<std::int32_t> s(L.s);
    std::vector<ex::RowA8> table;
    for (std::uint32_t t = 0; t < T; ++t) table.push_back(ex::RowA8{c.p + t * H, d.p + t * (H / 32), s.p + t * (H / 32)});
    std::vector<ex::Assignment> list;
    for (std::uint32_t t = T; t-- > 0;)                      // rows in descending order: the list is in no particular order
        for (std::uint32_t k = 0; k < K; ++k) list.push_back(ex::Assignment{t, k, L.routes[t * K + k]});
    Dev<ex::RowA8> dtable(table);
    Dev<ex::Assignment> dlist(list);
    const std::uint64_t row_stride = K * H + 32;
    Dev<float> raw(T * row_stride);
    Dev<std::uint32_t> status(T);
    ex::Job job;
    job.weights = ex::LayerWeights{gate.p, up.p, down.p, ex::GateFormat::q4_k, ex::DownFormat::q8_0, ex::Shape{H, I}};
    job.rows = dtable.p; job.assignments = dlist.p; job.count = static_cast<std::uint32_t>(list.size());
    job.rawdots = raw.p; job.rawdot_row_stride = row_stride; job.status = status.p;
    ex::Executor pool(64, 256);
    pool.run(job);
    const std::vector<float> got = raw.get();
    bool ok = true;
    for (std::uint32_t t = 0; t < T; ++t) ok = ok && std::memcmp(got.data() + t * row_stride, ref.rawdots.data() + size_t(t) * K * H, 4 * K * H) == 0;
    expect(ok && status.get() == std::vector<std::uint32_t>(T, 0U), "expert::Executor::run(Job): rawdots == oracle");
    bool threw = false;
    job.count = 65;
    try { pool.run(job); } catch (const std::invalid_argument&) { threw = true; }
    expect(threw, "expert::Executor::run throws std::invalid_argument for a job beyond its capacity");
}

int main() {
    int devices = 0;
    if (hipGetDeviceCount(&devices) != hipSuccess || devices == 0) { std::printf("no GPU\n"); return 99; }
    hip(hipSetDevice(0), "hipSetDevice");
    try {
        kernel_table();
        weight_runtime();
        const Layer L;
        a8_single_row(L);
        a8_serial_forms(L);
        combine_forms();
        a8_union_rows(L);
        strided_rows(L);
        executor_job(L);
    } catch (const std::exception& e) {
        std::printf("FAIL exception: %s\n", e.what());
        return 98;
    }
    hip(hipDeviceSynchronize(), "hipDeviceSynchronize");
    std::printf("%d failed\n", failures);
    return failures;
}
