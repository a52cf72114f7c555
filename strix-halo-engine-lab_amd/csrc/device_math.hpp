// Device-side scalar arithmetic shared by every kernel of the library: conversions, the two exp forms, cross-lane
// moves. Every float operation is a single IEEE binary32 round-to-nearest operation; the translation unit is built
// with -ffp-contract=off so no multiply-add is fused unless fmaf() is written.
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace strix950 {

// Plain 128-bit register values. (HIP's uint4 / float4 are structs whose whole-value copies lower to memcpy, which can
// pin an array of them in scratch memory; these vector types always live in VGPRs.)
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float f_of(uint32_t b) { return __builtin_bit_cast(float, b); }
__device__ __forceinline__ uint32_t b_of(float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ __forceinline__ bool finite_f(float x) { return (b_of(x) & 0x7f800000U) != 0x7f800000U; }

// fp16 bits -> fp32, exact for every value (subnormals included). Reference: src/cpu/core/reference.cpp:15-24.
__device__ __forceinline__ float half_bits_to_float(uint32_t h) {
    return __half2float(__ushort_as_half(static_cast<unsigned short>(h)));
}
// fp32 -> fp16 bits, round to nearest even, by integer arithmetic (the weight writers' scale conversion).
__device__ __forceinline__ uint32_t float_to_half_bits(float value) {
    uint32_t x = b_of(value);
    const uint32_t sign = (x >> 16) & 0x8000U;
    x &= 0x7fffffffU;
    if (x >= 0x7f800000U) return sign | 0x7c00U | (x > 0x7f800000U ? 0x200U | ((x >> 13) & 0x3ffU) : 0U);
    if (x >= 0x477ff000U) return sign | 0x7c00U;
    if (x < 0x38800000U) {
        if (x <= 0x33000000U) return sign;
        const uint32_t e = x >> 23, m = (x & 0x7fffffU) | 0x800000U, shift = 126U - e;
        uint32_t r = m >> shift;
        const uint32_t rem = m & ((1U << shift) - 1U), half = 1U << (shift - 1U);
        if (rem > half || (rem == half && (r & 1U))) ++r;
        return sign | r;
    }
    uint32_t h = (x - 0x38000000U) >> 13;
    const uint32_t rem = x & 0x1fffU;
    if (rem > 0x1000U || (rem == 0x1000U && (h & 1U))) ++h;
    return sign | h;
}

template <int KIND> __device__ __forceinline__ float load_activation(const void* row, uint32_t i);
template <> __device__ __forceinline__ float load_activation<0>(const void* row, uint32_t i) { return static_cast<const float*>(row)[i]; }
template <> __device__ __forceinline__ float load_activation<1>(const void* row, uint32_t i) {
    return half_bits_to_float(static_cast<const unsigned short*>(row)[i]);
}
template <> __device__ __forceinline__ float load_activation<2>(const void* row, uint32_t i) {
    return f_of(static_cast<uint32_t>(static_cast<const unsigned short*>(row)[i]) << 16);
}
__device__ __forceinline__ float load_activation_kind(const void* row, uint32_t i, uint32_t kind) {
    return kind == 0 ? load_activation<0>(row, i) : kind == 1 ? load_activation<1>(row, i) : load_activation<2>(row, i);
}

// exp(x) from basic IEEE operations only, the same bits on host and device. Reference: include/strix/ds41_moe.hpp:38-54.
__device__ __forceinline__ float declared_exp(float x) {
    if (!(x == x)) return x;
    if (x > 88.0F) return f_of(0x7f800000U);
    if (x < -103.0F) return 0.0F;
    const float n = __builtin_rintf(x * 1.44269504F);
    const float r = (x - n * 0.693359375F) - n * -2.12194440e-4F;
    float p = 1.98412698e-4F;
    p = p * r + 1.38888889e-3F;
    p = p * r + 8.33333333e-3F;
    p = p * r + 4.16666667e-2F;
    p = p * r + 1.66666667e-1F;
    p = p * r + 0.5F;
    p = p * r + 1.0F;
    p = p * r + 1.0F;
    const int k = static_cast<int>(n), k1 = k / 2, k2 = k - k1;
    return (p * f_of(static_cast<uint32_t>(k1 + 127) << 23)) * f_of(static_cast<uint32_t>(k2 + 127) << 23);
}

// The host twin of the gfx1151 expf with no probe-table corrections: Cody-Waite split of x * log2(e), then
// 2^a for |a| < 1 as the float rounding of a double-precision exp2, scaled by 2^e.
// Reference: src/cpu/core/routed_expert.cpp:212-216,248-261.
__device__ __forceinline__ float expf_gfx1151(float x) {
    const float kLog2e = f_of(0x3fb8aa3bU), kLog2eLo = f_of(0x32a5705fU);
    const float ph = x * kLog2e;
    const float e = __builtin_rintf(ph);
    float pl = __builtin_fmaf(x, kLog2e, -ph);
    pl = __builtin_fmaf(x, kLog2eLo, pl);
    const float a = (ph - e) + pl;
    float y;
    if (__builtin_fabsf(a) < 1.0F) y = __builtin_ldexpf(static_cast<float>(exp2(static_cast<double>(a))), static_cast<int>(e));
    else y = a != a ? a : 0.0F;
    if (f_of(0xc2ce8ed0U) > x) y = 0.0F;
    if (f_of(0x42b17218U) < x) y = f_of(0x7f800000U);
    return y;
}
// The C library's single-precision exp as the reference's router test oracle calls it (std::exp on a float,
// tests/hip_moe_route_launcher_tests.hip:329): z = x * 32 / ln 2 in double, k = round(z) by the 1.5 * 2^52 shift, r = z - k,
// 2^(k / 32) from a 32-entry table with k's upper bits added to the exponent, a cubic in r, one rounding to float.
// Every operation is a double-precision IEEE operation, so the bits are the host library's wherever its own result is
// not within a few double ulps of a float rounding boundary.
__device__ __forceinline__ float expf_libm(float x) {
    static constexpr unsigned long long kTab[32] = {
        0x3ff0000000000000ULL, 0x3fefd9b0d3158574ULL, 0x3fefb5586cf9890fULL, 0x3fef9301d0125b51ULL,
        0x3fef72b83c7d517bULL, 0x3fef54873168b9aaULL, 0x3fef387a6e756238ULL, 0x3fef1e9df51fdee1ULL,
        0x3fef06fe0a31b715ULL, 0x3feef1a7373aa9cbULL, 0x3feedea64c123422ULL, 0x3feece086061892dULL,
        0x3feebfdad5362a27ULL, 0x3feeb42b569d4f82ULL, 0x3feeab07dd485429ULL, 0x3feea47eb03a5585ULL,
        0x3feea09e667f3bcdULL, 0x3fee9f75e8ec5f74ULL, 0x3feea11473eb0187ULL, 0x3feea589994cce13ULL,
        0x3feeace5422aa0dbULL, 0x3feeb737b0cdc5e5ULL, 0x3feec49182a3f090ULL, 0x3feed503b23e255dULL,
        0x3feee89f995ad3adULL, 0x3feeff76f2fb5e47ULL, 0x3fef199bdd85529cULL, 0x3fef3720dcef9069ULL,
        0x3fef5818dcfba487ULL, 0x3fef7c97337b9b5fULL, 0x3fefa4afa2a490daULL, 0x3fefd0765b6e4540ULL};
    if (!(x == x)) return x + x;
    if (x > 0x1.62e42ep6F) return f_of(0x7f800000U);
    if (x < -0x1.9fe368p6F) return 0.0F;
    const double z = (0x1.71547652b82fep+0 * 32.0) * static_cast<double>(x);
    double kd = z + 0x1.8p+52;
    const unsigned long long ki = __builtin_bit_cast(unsigned long long, kd);
    kd = kd - 0x1.8p+52;
    const double r = z - kd;
    const double s = __builtin_bit_cast(double, kTab[ki % 32U] + (ki << 47));
    const double c01 = (0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0) * r + (0x1.ebfce50fac4f3p-3 / 32.0 / 32.0);
    const double r2 = r * r;
    double y = (0x1.62e42ff0c52d6p-1 / 32.0) * r + 1.0;
    y = c01 * r2 + y;
    y = y * s;
    return static_cast<float>(y);
}
__device__ __forceinline__ float exp_of(uint32_t kind, float x) { return kind == 1U ? declared_exp(x) : kind == 2U ? expf_libm(x) : expf_gfx1151(x); }

// The SwiGLU clamp trait (include/strix/moe/activation_policy.hpp:22-24): gate from above, up on both sides; NaN passes
// through; limit = +infinity clamps nothing (every comparison is false).
__device__ __forceinline__ void swiglu_clamp(float& g, float& u, float limit) {
    g = g > limit ? limit : g;
    u = u < -limit ? -limit : (u > limit ? limit : u);
}

// A store that another workgroup of the same launch reads (device scope: performed at the memory side, past the per-XCD
// caches), or a plain one.
template <class T>
__device__ __forceinline__ void store_shared_or_plain(bool device_scope, T* p, T v) {
    if (device_scope) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else *p = v;
}

// ---- cross-lane moves inside a 64-wide wavefront ----------------------------------------------------------------
// lane ^ 1 and lane ^ 2 are DPP quad permutes (no LDS traffic); wider distances go through the swizzle crossbar.
__device__ __forceinline__ int xor1_i(int v) { return __builtin_amdgcn_mov_dpp(v, 0xB1, 0xF, 0xF, true); }
__device__ __forceinline__ int xor2_i(int v) { return __builtin_amdgcn_mov_dpp(v, 0x4E, 0xF, 0xF, true); }
// lane ^ 4 inside a group of 8: mirror the 8 lanes (row_half_mirror), then reverse each quad - two DPP moves.
__device__ __forceinline__ int xor4_i(int v) { return __builtin_amdgcn_mov_dpp(__builtin_amdgcn_mov_dpp(v, 0x141, 0xF, 0xF, true), 0x1B, 0xF, 0xF, true); }
__device__ __forceinline__ int xor8_i(int v) { return __builtin_amdgcn_ds_swizzle(v, 0x201F); }
__device__ __forceinline__ int xor16_i(int v) { return __builtin_amdgcn_ds_swizzle(v, 0x401F); }
__device__ __forceinline__ float xor1_f(float v) { return __builtin_bit_cast(float, xor1_i(__builtin_bit_cast(int, v))); }
__device__ __forceinline__ float xor2_f(float v) { return __builtin_bit_cast(float, xor2_i(__builtin_bit_cast(int, v))); }
__device__ __forceinline__ float xor4_f(float v) { return __builtin_bit_cast(float, xor4_i(__builtin_bit_cast(int, v))); }
__device__ __forceinline__ float xor8_f(float v) { return __builtin_bit_cast(float, xor8_i(__builtin_bit_cast(int, v))); }
__device__ __forceinline__ float xor16_f(float v) { return __builtin_bit_cast(float, xor16_i(__builtin_bit_cast(int, v))); }

// Reductions over an aligned group of 32 lanes (a half wavefront). max and integer sums are order-free.
__device__ __forceinline__ float max32(float v) {
    v = __builtin_fmaxf(v, xor1_f(v)); v = __builtin_fmaxf(v, xor2_f(v)); v = __builtin_fmaxf(v, xor4_f(v));
    v = __builtin_fmaxf(v, xor8_f(v)); v = __builtin_fmaxf(v, xor16_f(v));
    return v;
}
__device__ __forceinline__ int sum32_i(int v) {
    v += xor1_i(v); v += xor2_i(v); v += xor4_i(v); v += xor8_i(v); v += xor16_i(v);
    return v;
}
__device__ __forceinline__ int or32_i(int v) {
    v |= xor1_i(v); v |= xor2_i(v); v |= xor4_i(v); v |= xor8_i(v); v |= xor16_i(v);
    return v;
}

// A8 code of one value under a group delta. Reference: src/cpu/core/reference.cpp:47-48.
__device__ __forceinline__ int a8_code(float x, float delta, bool tiny) {
    const float rounded = tiny ? 0.0F : __builtin_rintf(x / delta);
    const float lo = -127.0F < rounded ? rounded : -127.0F;
    const float cl = lo < 127.0F ? lo : 127.0F;
    return static_cast<int>(cl);
}

}  // namespace strix950
