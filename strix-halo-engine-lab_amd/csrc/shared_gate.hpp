// The scalar gate of an always-on shared expert: gate[row] = 1 / (1 + exp(-dot(x[row], scalar_weight))), the weight its output
// carries into the layer's sum (tensor ffn_gate_inp_shexp, F32 [hidden]).
// Reference: src/hip_shared_expert_launcher.hip:624-645 (shared_gate_dot / rows_shared_gate_dot_kernel; the same body at :586-594 and
// :616-621) with the tree of src/core/ordered_reduce.hpp:8-16,46-67:
//   one workgroup of 256 threads per row; thread t: sum = 0, then sum += x[f] * w[f] for f = t, t + 256, ... in ascending f.
//     The reference's library target sets no contraction flag for this file, so the device compiler's default fuses the
//     statement: each step is one fma(x[f], w[f], sum);
//   the 256 partial sums go through the halving tree s[l] = s[l] + s[l + h], h = 128, 64, ..., 1 (own + partner, one IEEE add);
//   gate = 1 / (1 + expf(-dot)) with the device expf (the SiLU's exp of the same launcher) and a correctly rounded division.
#pragma once

namespace strix950 {

template <int KIND>
__global__ __launch_bounds__(256) void shared_gate_kernel(const uint8_t* x, uint64_t x_stride, uint32_t hidden, const float* weight, uint32_t exp_kind,
                                                          float* gate, uint64_t gate_stride) {
    __shared__ float s[256];
    const uint32_t t = threadIdx.x, row = blockIdx.x;
    const uint8_t* xr = x + row * x_stride;
    float sum = 0.0F;
#pragma unroll 8
    for (uint32_t f = t; f < hidden; f += 256U) sum = __builtin_fmaf(load_activation<KIND>(xr, f), weight[f], sum);
    s[t] = sum;
    __syncthreads();
#pragma unroll
    for (uint32_t h = 128U; h >= 1U; h >>= 1) {
        if (t < h) s[t] = s[t] + s[t + h];
        __syncthreads();
    }
    if (t == 0) gate[row * gate_stride] = 1.0F / (1.0F + exp_of(exp_kind, -s[0]));
}

}  // namespace strix950

extern "C" {

int32_t mi355_shared_gate(const void* x, uint32_t input_kind, uint32_t rows, uint32_t hidden, uint64_t x_stride_bytes, const float* scalar_weight,
                          uint32_t exp_kind, float* gate, uint64_t gate_stride, mi355_stream stream) {
    using namespace strix950;
    if (rows == 0) return MI355_OK;
    STRIX_REQUIRE(x && scalar_weight && gate && hidden > 0, "shared gate: null pointer or empty row");
    STRIX_REQUIRE(input_kind <= MI355_INPUT_BF16 && exp_kind <= MI355_EXP_LIBM, "shared gate: unknown input or exp kind");
    const uint32_t unit = input_kind == MI355_INPUT_F32 ? 4U : 2U;
    STRIX_REQUIRE(aligned(x, unit) && x_stride_bytes % unit == 0 && x_stride_bytes >= static_cast<uint64_t>(hidden) * unit && aligned(scalar_weight, 4) &&
                  aligned(gate, 4) && gate_stride >= 1, "shared gate: views must be element-aligned with strides that cover a row");
    STRIX_REQUIRE(rows <= 0x7fffffffU, "shared gate: too many rows");
    const uint8_t* xb = static_cast<const uint8_t*>(x);
    hipStream_t st = hs(stream);
    if (input_kind == MI355_INPUT_F32) shared_gate_kernel<0><<<rows, 256, 0, st>>>(xb, x_stride_bytes, hidden, scalar_weight, exp_kind, gate, gate_stride);
    else if (input_kind == MI355_INPUT_F16) shared_gate_kernel<1><<<rows, 256, 0, st>>>(xb, x_stride_bytes, hidden, scalar_weight, exp_kind, gate, gate_stride);
    else shared_gate_kernel<2><<<rows, 256, 0, st>>>(xb, x_stride_bytes, hidden, scalar_weight, exp_kind, gate, gate_stride);
    STRIX_LAUNCHED("shared gate");
    return MI355_OK;
}

}  // extern "C"
