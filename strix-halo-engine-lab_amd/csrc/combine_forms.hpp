// The combine as an operator of its own: y[row][d] = ordered reduction of eo[row][0..top_k)[d] with the route weights, plus a
// base. Reference: the host restatement include/strix/moe/combine.hpp:36-59 and the device operator
// src/moe_core/route_wave_kernel.hpp:98-160 (enqueue_combine, enqueue_combine_rounded_eo).
//   fma form:        acc = fma(w_k, e_k, acc) over the slots in order, y = acc + base                (weights and base required)
//   bf16-steps form: acc = bf16(acc + term_k), term_k = w ? bf16(e_k * w_k) : e_k;  y = base ? bf16(acc + base) : acc
//                    (bf16() = round to nearest even of the upper 16 bits, a NaN passes through untouched);
//                    with round_eo every e_k is first replaced by bf16(e_k).
// HBM-bound: (top_k + base + 1) * 4 bytes per output value; every slot's value is requested before the chain starts.
#pragma once

namespace strix950 {

__device__ __forceinline__ float combine_bf16(float x) {
    const uint32_t bits = __builtin_bit_cast(uint32_t, x);
    if ((bits & 0x7f800000U) == 0x7f800000U && (bits & 0x7fffffU)) return x;
    return __builtin_bit_cast(float, (bits + 0x7fffU + ((bits >> 16U) & 1U)) & 0xffff0000U);
}

struct CombineArgs {
    const float* w; const float* eo; const float* base; float* y;
    uint32_t top_k, width;
    uint64_t w_stride, eo_stride, base_stride, y_stride;     // floats per row
};

template <int VEC, int FORM, bool ROUND_EO>
__global__ __launch_bounds__(256) void combine_kernel(CombineArgs a) {
    typedef float vec_t __attribute__((ext_vector_type(VEC)));
    const uint32_t row = blockIdx.y, d = (blockIdx.x * 256U + threadIdx.x) * VEC;
    if (d >= a.width) return;
    const float* eo = a.eo + row * a.eo_stride + d;
    const float* w = a.w ? a.w + row * a.w_stride : nullptr;
    vec_t acc = 0.0F;
    for (uint32_t k0 = 0; k0 < a.top_k; k0 += 16U) {
        vec_t e[16];
        float wk[16];
#pragma unroll
        for (uint32_t k = 0; k < 16U; ++k)
            if (k0 + k < a.top_k) {
                e[k] = *reinterpret_cast<const vec_t*>(eo + static_cast<size_t>(k0 + k) * a.width);
                wk[k] = w ? w[k0 + k] : 1.0F;
            }
#pragma unroll
        for (uint32_t k = 0; k < 16U; ++k) {
            if (k0 + k >= a.top_k) continue;
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
                if constexpr (FORM == MI355_COMBINE_FMA_SLOT_ORDER) {
                    acc[c] = __builtin_fmaf(wk[k], e[k][c], acc[c]);
                } else {
                    const float ev = ROUND_EO ? combine_bf16(e[k][c]) : e[k][c];
                    const float term = w ? combine_bf16(ev * wk[k]) : ev;
                    acc[c] = combine_bf16(acc[c] + term);
                }
            }
        }
    }
    if (a.base) {
        const vec_t b = *reinterpret_cast<const vec_t*>(a.base + row * a.base_stride + d);
#pragma unroll
        for (int c = 0; c < VEC; ++c) acc[c] = FORM == MI355_COMBINE_FMA_SLOT_ORDER ? acc[c] + b[c] : combine_bf16(acc[c] + b[c]);
    }
    *reinterpret_cast<vec_t*>(a.y + row * a.y_stride + d) = acc;
}

template <int FORM, bool ROUND_EO>
void launch_combine(const CombineArgs& a, uint32_t rows, bool quads, hipStream_t st) {
    if (quads) combine_kernel<4, FORM, ROUND_EO><<<dim3((a.width + 1023U) / 1024U, rows), 256, 0, st>>>(a);
    else combine_kernel<1, FORM, ROUND_EO><<<dim3((a.width + 255U) / 256U, rows), 256, 0, st>>>(a);
}

}  // namespace strix950

extern "C" {

int32_t mi355_moe_enqueue_combine(uint32_t form, uint32_t rows, uint32_t top_k, uint32_t width, const float* w, const float* eo,
                                  const float* base, float* y, uint32_t round_eo, mi355_stream stream) {
    using namespace strix950;
    STRIX_REQUIRE(form == MI355_COMBINE_FMA_SLOT_ORDER || form == MI355_COMBINE_BF16_STEPS, "moe combine: form must be the fma or the bf16-steps one");
    STRIX_REQUIRE(top_k > 0 && width > 0, "moe combine: top_k and width must be positive");        // combine.hpp:41
    STRIX_REQUIRE(rows <= 65535U, "moe combine: at most 65535 rows per call");
    if (form == MI355_COMBINE_FMA_SLOT_ORDER) {
        STRIX_REQUIRE(w && base, "moe combine: fma_f32 needs weights and base");                    // combine.hpp:44, route_wave_kernel.hpp:146
        STRIX_REQUIRE(!round_eo, "moe combine: rounded operands are bound for the bf16-steps form only");   // route_wave_kernel.hpp:103
    }
    if (rows == 0U) return MI355_OK;                                                               // route_wave_kernel.hpp:147
    STRIX_REQUIRE(eo && y, "moe combine: null operand or output");
    STRIX_REQUIRE(aligned(eo, 4) && aligned(y, 4) && aligned(w, 4) && aligned(base, 4), "moe combine: views must be float-aligned");
    const CombineArgs a{w, eo, base, y, top_k, width, top_k, static_cast<uint64_t>(top_k) * width, width, width};
    const bool quads = width % 4U == 0 && aligned(eo, 16) && aligned(y, 16) && (!base || aligned(base, 16)) &&
                       static_cast<uint64_t>(rows) * ((width + 1023U) / 1024U) >= 4ULL * compute_units();
    hipStream_t st = hs(stream);
    if (form == MI355_COMBINE_FMA_SLOT_ORDER) launch_combine<MI355_COMBINE_FMA_SLOT_ORDER, false>(a, rows, quads, st);
    else if (round_eo) launch_combine<MI355_COMBINE_BF16_STEPS, true>(a, rows, quads, st);
    else launch_combine<MI355_COMBINE_BF16_STEPS, false>(a, rows, quads, st);
    STRIX_LAUNCHED("moe combine");
    return MI355_OK;
}

}  // extern "C"
