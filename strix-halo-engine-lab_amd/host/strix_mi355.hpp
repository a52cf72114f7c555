// Header-only C++ mirror of the engine-side interfaces this library replaces, over the C ABI in mi355_strix.h.
// Same names, argument meaning and error behaviour as the reference, so host code written against the reference reads
// unchanged:
//   strix::mi355::Q8a8View / Kernels         <- strix::cpu::Q8a8View / Kernels   (src/cpu/core/backend.hpp:52-73)
//   strix::mi355::qwen_moe::Rows / Weights / enqueue_prologue .. enqueue_merge / enqueue
//                                             <- strix::cuda::qwen_moe          (include/strix/cuda/qwen_moe.hpp:55-110)
//   strix::mi355::moe_route::enqueue          <- the route launcher              (include/strix/hip_moe_route_launcher.hpp:16-30)
// Admission failures throw std::invalid_argument before anything is enqueued, HIP failures throw std::runtime_error, as
// the reference's validate() / hip_check do. Every pointer is device memory; nothing here allocates or synchronises.
#pragma once
#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>

#include "mi355_strix.h"

namespace strix::mi355 {

inline void check(std::int32_t rc) {
    if (rc == MI355_OK) return;
    const std::string why = mi355_last_error();
    if (rc == MI355_E_INVALID_ARGUMENT || rc == MI355_E_UNSUPPORTED) throw std::invalid_argument(why);
    throw std::runtime_error(why);
}

// ---------------------------------------------------------------------------------------------- dense kernel table
using Q8a8View = mi355_q8a8_view;                       // field for field strix::cpu::Q8a8View
struct Stream { mi355_stream stream = nullptr; };       // the reference's Stream carries a thread count; here a HIP stream

struct Kernels {
    // x: device fp32 [width]. Throws std::invalid_argument for width % 32 != 0 before any write; sums may be null.
    static void quantize_a8(const float* x, std::size_t width, std::int8_t* codes, float* deltas, std::int32_t* sums,
                            const Stream& s = {}) {
        check(mi355_quantize_a8(x, MI355_INPUT_F32, 1, static_cast<std::uint32_t>(width), width * sizeof(float), codes, deltas,
                                sums, nullptr, s.stream));
    }
    static void gemv_q8_0_a8(const Q8a8View& v, const Stream& s = {}) { check(mi355_gemv_q8_0_a8(&v, s.stream)); }
    // x, y: device fp32 [rows][n]; w: device fp32 [n] or null (the signature of strix::cpu::Kernels::rmsnorm_f32)
    static void rmsnorm_f32(const float* x, const float* w, unsigned n, float eps, float* y, unsigned rows, const Stream& s = {}) {
        check(mi355_rmsnorm_f32(x, w, n, eps, y, rows, s.stream));
    }
};

// ---------------------------------------------------------------------------------------------- router
namespace moe_route {
using Policy = mi355_route_policy;
inline void enqueue(const Policy& policy, const void* x, std::uint32_t input_kind, std::uint32_t rows, std::uint32_t hidden,
                    std::uint64_t x_stride_bytes, const float* router_weight, const float* logit_bias, std::uint32_t* ids,
                    float* weights, float* scores, mi355_stream stream) {
    check(mi355_moe_route(&policy, x, input_kind, rows, hidden, x_stride_bytes, router_weight, logit_bias, ids, weights, scores,
                          stream));
}
}  // namespace moe_route

// ---------------------------------------------------------------------------------------------- routed experts
namespace qwen_moe {
using Rows = mi355_moe_rows;          // per-row views: input, routes, route_weights, A8 image, status, h image, rawdots, output
using Weights = mi355_moe_weights;    // gate / up [experts][ffn][hidden/256 blocks], down [experts][hidden][ffn/256 blocks]

inline std::size_t plan_words(std::uint32_t experts, std::uint32_t rows, std::uint32_t top_k) {
    return mi355_moe_plan_words(experts, rows, top_k);
}
inline std::size_t prefill_f16_workspace_bytes(std::uint32_t hidden, std::uint32_t ffn, std::uint32_t rows, std::uint32_t top_k) {
    return mi355_moe_prefill_f16_workspace_bytes(hidden, ffn, rows, top_k);
}
inline void enqueue_prologue(const Rows& r, std::uint32_t rows, const Weights& w, mi355_stream s) { check(mi355_moe_enqueue_prologue(&w, &r, rows, s)); }
inline void enqueue_csr(const Rows& r, std::uint32_t rows, const Weights& w, mi355_stream s) { check(mi355_moe_enqueue_csr(&w, &r, rows, s)); }
inline void enqueue_project(const Rows& r, std::uint32_t rows, const Weights& w, mi355_stream s) { check(mi355_moe_enqueue_project(&w, &r, rows, s)); }
inline void enqueue_down(const Rows& r, std::uint32_t rows, const Weights& w, mi355_stream s) { check(mi355_moe_enqueue_down(&w, &r, rows, s)); }
inline void enqueue_merge(const Rows& r, std::uint32_t rows, const Weights& w, mi355_stream s,
                          std::uint32_t form = MI355_COMBINE_FMA_SLOT_ORDER) {
    check(mi355_moe_enqueue_merge(&w, &r, rows, form, s));
}
// prologue + csr + project + down + merge
inline void enqueue(const Rows& r, std::uint32_t rows, const Weights& w, mi355_stream s,
                    std::uint32_t form = MI355_COMBINE_FMA_SLOT_ORDER) {
    check(mi355_moe_enqueue(&w, &r, rows, form, s));
}
// the routed experts of a prefill batch on fp16 MFMA (FAST class: follows the exact-weight product to 2e-3, not the
// integer-dot bits); needs r.h_f16 and fp16 input rows
inline void enqueue_prefill_f16(const Rows& r, std::uint32_t rows, const Weights& w, mi355_stream s,
                                std::uint32_t form = MI355_COMBINE_FMA_SLOT_ORDER) {
    check(mi355_moe_enqueue_prefill_f16(&w, &r, rows, form, s));
}
// router + the layer; r.routes / r.route_weights receive the selection
inline void enqueue_layer(const moe_route::Policy& policy, const float* router_weight, const float* logit_bias, float* scores,
                          const Rows& r, std::uint32_t rows, const Weights& w, mi355_stream s,
                          std::uint32_t form = MI355_COMBINE_FMA_SLOT_ORDER) {
    check(mi355_moe_enqueue_layer(&policy, router_weight, logit_bias, scores, &w, &r, rows, form, s));
}
}  // namespace qwen_moe

// SwiGLU + A8 re-quantisation of dense gate | up rows (enqueue_down_activation_quantize, include/strix/hip_moe_a8_down.hpp:18).
inline void enqueue_down_activation_quantize(const float* gate, const float* up, std::uint32_t rows, std::uint32_t ffn,
                                             std::uint32_t exp_kind, float swiglu_limit, std::int8_t* codes, float* deltas,
                                             std::int32_t* sums, float* h_out, std::uint32_t* status, mi355_stream s) {
    check(mi355_swiglu_quantize(gate, up, rows, ffn, exp_kind, swiglu_limit, codes, deltas, sums, h_out, status, s));
}

}  // namespace strix::mi355
