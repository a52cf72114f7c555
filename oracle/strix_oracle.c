/*
 * TEST INFRASTRUCTURE - CPU parity oracle (see strix_oracle.h). Never linked into the GPU library.
 * Build: gcc -O2 -std=c11 -ffp-contract=off -fno-fast-math -fopenmp -fPIC -shared.
 * All paths cited are relative to the reference tree.
 */
#include "strix_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#if defined(__FAST_MATH__)
#error "the oracle needs strict IEEE semantics"
#endif

static inline uint32_t bits_of(float f) { uint32_t b; memcpy(&b, &f, 4); return b; }
static inline float float_of(uint32_t b) { float f; memcpy(&f, &b, 4); return f; }
static inline int is_finite(float x) { return (bits_of(x) & 0x7f800000U) != 0x7f800000U; }
static inline uint16_t le16(const uint8_t* p) { return (uint16_t)(p[0] | ((unsigned)p[1] << 8)); }
static inline uint32_t le32(const uint8_t* p) { uint32_t v; memcpy(&v, p, 4); return v; }

/* Plain multi-thread read of a buffer (sum of its 64-bit words), seconds for `reps` passes: the host's memory-read ceiling
 * next to the CPU baseline (method of the reference's scripts/bench/residency/cpu_expert_bench.cpp:131-147). */
double orc_read_seconds(const uint64_t* buffer, size_t words, int reps, int threads, uint64_t* checksum) {
    uint64_t total = 0;
    const double t0 = omp_get_wtime();
    for (int r = 0; r < reps; ++r) {
        uint64_t sum = 0;
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static) reduction(+ : sum)
        for (size_t i = 0; i < words; ++i) sum += buffer[i];
        total += sum;
    }
    const double t1 = omp_get_wtime();
    if (checksum) *checksum = total;
    return t1 - t0;
}

int orc_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------ conversions */
/* src/cpu/core/reference.cpp:15-24: sign, subnormals via ldexp(mantissa, -24), inf/nan payload kept. */
float orc_half_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000U) << 16, e = (h >> 10) & 31U, m = h & 1023U;
    if (e == 0) { const float v = ldexpf((float)m, -24); return sign ? -v : v; }
    if (e == 31) return float_of(sign | 0x7f800000U | (m << 13));
    return float_of(sign | ((e + 112U) << 23) | (m << 13));
}

uint16_t orc_float_to_half(float value) {
    uint32_t x = bits_of(value);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000U);
    x &= 0x7fffffffU;
    if (x >= 0x7f800000U) return (uint16_t)(sign | 0x7c00U | (x > 0x7f800000U ? 0x200U | ((x >> 13) & 0x3ffU) : 0U));
    if (x >= 0x477ff000U) return (uint16_t)(sign | 0x7c00U);          /* >= 65520 rounds to inf */
    if (x < 0x38800000U) {                                            /* below 2^-14: half subnormal */
        if (x <= 0x33000000U) return sign;                            /* <= 2^-25 rounds to zero (tie to even) */
        const uint32_t e = x >> 23, m = (x & 0x7fffffU) | 0x800000U, shift = 126U - e;
        uint32_t r = m >> shift;
        const uint32_t rem = m & ((1U << shift) - 1U), half = 1U << (shift - 1U);
        if (rem > half || (rem == half && (r & 1U))) ++r;
        return (uint16_t)(sign | r);
    }
    uint32_t h = (x - 0x38000000U) >> 13;
    const uint32_t rem = x & 0x1fffU;
    if (rem > 0x1000U || (rem == 0x1000U && (h & 1U))) ++h;
    return (uint16_t)(sign | h);
}

/* ------------------------------------------------------------------ block decode */
/* src/ggml_dequant.cpp:84-87 */
void orc_dequant_q8_0_row(const uint8_t* row, size_t n, float* out) {
    for (size_t b = 0; b < n / 32; ++b) {
        const uint8_t* x = row + b * ORC_Q8_0_BLOCK;
        const float d = orc_half_to_float(le16(x));
        for (int j = 0; j < 32; ++j) out[b * 32 + j] = (float)(int8_t)x[2 + j] * d;
    }
}

/* src/ggml_dequant.cpp:43-50 */
void orc_q4k_scale_min(const uint8_t* q, int j, uint8_t* d, uint8_t* m) {
    if (j < 4) { *d = q[j] & 63; *m = q[j + 4] & 63; }
    else { *d = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4)); *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4)); }
}

/* src/cpu/core/routed_expert.cpp:65-71 */
unsigned orc_q4k_factor_words(const uint8_t* hd, unsigned group, int minimum) {
    const uint32_t y = le32(hd + 4), z = le32(hd + 8), w = le32(hd + 12);
    const unsigned shift = 8U * (group & 3U);
    const unsigned a = (y >> shift) & 255U, b = (z >> shift) & 255U, c = (w >> shift) & 255U;
    if (group < 4U) return (minimum ? b : a) & 63U;
    return minimum ? (c >> 4U) | ((b >> 6U) << 4U) : (c & 15U) | ((a >> 6U) << 4U);
}

/* src/ggml_dequant.cpp:119-130: y = d1 * q - m1 with d1 = d * sc, m1 = dmin * m (two products, one subtract). */
void orc_dequant_q4_k_row(const uint8_t* row, size_t n, float* out) {
    for (size_t b = 0; b < n / 256; ++b) {
        const uint8_t* x = row + b * ORC_Q4_K_BLOCK;
        const uint8_t* q = x + 16;
        const float d = orc_half_to_float(le16(x)), mn = orc_half_to_float(le16(x + 2));
        float* y = out + b * 256;
        int is = 0;
        for (int j = 0; j < 256; j += 64) {
            uint8_t sc, m;
            orc_q4k_scale_min(x + 4, is + 0, &sc, &m); const float d1 = d * sc, m1 = mn * m;
            orc_q4k_scale_min(x + 4, is + 1, &sc, &m); const float d2 = d * sc, m2 = mn * m;
            for (int l = 0; l < 32; ++l) *y++ = d1 * (float)(q[l] & 0xF) - m1;
            for (int l = 0; l < 32; ++l) *y++ = d2 * (float)(q[l] >> 4) - m2;
            q += 32; is += 2;
        }
    }
}

/* ------------------------------------------------------------------ writers */
/* include/strix/q8_0_rule.hpp:25-33: d = amax / 127 (fp32), id = 1 / d, q = roundf(v * id); d stored as fp16. */
void orc_quantize_q8_0_row(const float* x, size_t n, uint8_t* out) {
    for (size_t b = 0; b < n / 32; ++b) {
        const float* v = x + b * 32;
        float amax = 0.0F;
        for (int j = 0; j < 32; ++j) amax = fmaxf(amax, fabsf(v[j]));
        const float d = amax / 127.0F;
        const float id = d != 0.0F ? 1.0F / d : 0.0F;
        uint8_t* o = out + b * ORC_Q8_0_BLOCK;
        const uint16_t h = orc_float_to_half(d);
        o[0] = (uint8_t)h; o[1] = (uint8_t)(h >> 8);
        for (int j = 0; j < 32; ++j) o[2 + j] = (uint8_t)(int8_t)(int)roundf(v[j] * id);
    }
}

/* A plain min/max Q4_K writer (no reference counterpart; the GPU writer restates the same steps):
 * per 32: lo = min(min x, 0), hi = max(max x, lo); scale = (hi - lo) / 15, offset = 0 - lo (never -0);
 * per 256: d = fp16(max scale / 63), dmin = fp16(max offset / 63); sc = min(63, rint(scale / d)),
 * m = min(63, rint(offset / dmin)); q = clamp(rint((x + dmin * m) / (d * sc)), 0, 15). */
void orc_quantize_q4_k_row(const float* x, size_t n, uint8_t* out) {
    for (size_t b = 0; b < n / 256; ++b) {
        const float* v = x + b * 256;
        uint8_t* o = out + b * ORC_Q4_K_BLOCK;
        float scale[8], offset[8], smax = 0.0F, omax = 0.0F;
        for (int j = 0; j < 8; ++j) {
            float lo = 0.0F, hi = v[32 * j];
            for (int l = 0; l < 32; ++l) { lo = fminf(lo, v[32 * j + l]); hi = fmaxf(hi, v[32 * j + l]); }
            hi = fmaxf(hi, lo);
            scale[j] = (hi - lo) / 15.0F; offset[j] = 0.0F - lo;
            smax = fmaxf(smax, scale[j]); omax = fmaxf(omax, offset[j]);
        }
        const uint16_t dh = orc_float_to_half(smax / 63.0F), mh = orc_float_to_half(omax / 63.0F);
        const float d = orc_half_to_float(dh), dm = orc_half_to_float(mh);
        uint8_t sc[8], mn[8];
        for (int j = 0; j < 8; ++j) {
            sc[j] = d > 0.0F ? (uint8_t)fminf(63.0F, rintf(scale[j] / d)) : 0;
            mn[j] = dm > 0.0F ? (uint8_t)fminf(63.0F, rintf(offset[j] / dm)) : 0;
        }
        o[0] = (uint8_t)dh; o[1] = (uint8_t)(dh >> 8); o[2] = (uint8_t)mh; o[3] = (uint8_t)(mh >> 8);
        for (int j = 0; j < 4; ++j) {
            o[4 + j] = (uint8_t)((sc[j] & 63) | ((sc[j + 4] >> 4) << 6));
            o[8 + j] = (uint8_t)((mn[j] & 63) | ((mn[j + 4] >> 4) << 6));
            o[12 + j] = (uint8_t)((sc[j + 4] & 15) | ((mn[j + 4] & 15) << 4));
        }
        uint8_t q[256];
        for (int j = 0; j < 8; ++j) {
            const float ed = d * (float)sc[j], em = dm * (float)mn[j];
            for (int l = 0; l < 32; ++l) {
                float r = 0.0F;
                if (ed > 0.0F) r = fminf(15.0F, fmaxf(0.0F, rintf((v[32 * j + l] + em) / ed)));
                q[32 * j + l] = (uint8_t)r;
            }
        }
        for (int p = 0; p < 4; ++p)
            for (int l = 0; l < 32; ++l) o[16 + 32 * p + l] = (uint8_t)(q[64 * p + l] | (q[64 * p + 32 + l] << 4));
    }
}

/* ------------------------------------------------------------------ A8 quantiser */
int orc_quantize_a8(const float* x, size_t width, int8_t* codes, float* deltas, int32_t* sums, int tiny_rule) {
    if (width % 32 != 0) return -1;
    int nonfinite = 0;
    for (size_t g = 0; g < width / 32; ++g) {
        const float* xg = x + g * 32;
        float amax = 0.0F;
        for (int j = 0; j < 32; ++j) {
            const float a = fabsf(xg[j]);
            if (!is_finite(xg[j])) nonfinite = 1;
            amax = amax < a ? a : amax;                     /* std::max(amax, |x|) */
        }
        const int tiny = tiny_rule && amax > 0.0F && amax < 0x1p-119F;
        const float delta = (amax == 0.0F || tiny) ? 1.0F : amax / 127.0F;
        int32_t sum = 0;
        for (int j = 0; j < 32; ++j) {
            const float rounded = tiny ? 0.0F : nearbyintf(xg[j] / delta);
            const float lo = -127.0F < rounded ? rounded : -127.0F;   /* std::max(-127, rounded) */
            const float cl = lo < 127.0F ? lo : 127.0F;               /* std::min(127, .) */
            const int8_t code = (int8_t)cl;
            codes[g * 32 + j] = code;
            sum += code;
        }
        deltas[g] = delta;
        if (sums) sums[g] = sum;
    }
    return nonfinite;
}

/* ------------------------------------------------------------------ Q8_0 x A8 */
static float tree32(float* v) {   /* src/core/integer_math.hpp:43-47 */
    for (unsigned s = 16; s; s /= 2)
        for (unsigned i = 0; i < s; ++i) v[i] = v[i] + v[i + s];
    return v[0];
}

int orc_gemv_q8_0_a8(const orc_q8a8_view* v, int threads) {
    if (v->in % 32 != 0) return -1;
    const size_t groups = v->in / 32;
    for (uint32_t r = 0; r < v->rows; ++r) {
        const int8_t* xc = v->codes + (size_t)r * v->x_stride;
        const float* xd = v->deltas + (size_t)r * (v->x_stride / 32);
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
        for (uint32_t o = 0; o < v->count; ++o) {
            float lanes[32];
            for (int i = 0; i < 32; ++i) lanes[i] = 0.0F;
            for (size_t g = 0; g < groups; ++g) {
                const uint8_t* block = v->weight + (size_t)o * v->row_bytes + g * ORC_Q8_0_BLOCK;
                const float scale = orc_half_to_float(le16(block));
                int32_t dot = 0;
                for (int j = 0; j < 32; ++j) dot += (int)(int8_t)block[2 + j] * (int)xc[g * 32 + j];
                /* product(dot, sw, sa) = float(dot) * (sw * sa) */
                lanes[g % 32] = lanes[g % 32] + (float)dot * (scale * xd[g]);
            }
            float* y = &v->out[(size_t)r * v->out_stride + o];
            const float p = tree32(lanes);
            *y = v->accumulate ? *y + p : p;
        }
    }
    return 0;
}

/* ------------------------------------------------------------------ RMSNorm */
/* src/cpu/core/reference.cpp:86-103; lane count src/cpu/core/backend.hpp:91. */
void orc_rmsnorm_f32(const float* x, const float* w, uint32_t n, float eps, float* y, uint32_t rows) {
    const uint32_t lanes = n >= 512 ? 256U : 128U;
    float partial[256];
    for (uint32_t row = 0; row < rows; ++row) {
        const float* xr = x + (size_t)row * n;
        float* yr = y + (size_t)row * n;
        for (uint32_t lane = 0; lane < lanes; ++lane) {
            float a = 0.0F;
            for (uint32_t i = lane; i < n; i += lanes) a = fmaf(xr[i], xr[i], a);
            partial[lane] = a;
        }
        for (uint32_t h = lanes / 2; h > 0; h >>= 1)
            for (uint32_t lane = 0; lane < h; ++lane) partial[lane] = partial[lane] + partial[lane + h];
        const float r = 1.0F / sqrtf(partial[0] / (float)n + eps);
        for (uint32_t i = 0; i < n; ++i) yr[i] = w ? (xr[i] * r) * w[i] : xr[i] * r;
    }
}

/* ------------------------------------------------------------------ Q4_K x A8 row */
/* The exact int32 group dots of one super-block (dot[j] = sum_k code * nibble, sub-block j = 2p low / 2p + 1 high nibbles of
 * bytes 32p .. 32p + 31). Integer arithmetic only, so the compiler may vectorise it for whatever the host offers (the clones
 * are picked at load time); the fp32 chain around it stays scalar and in the declared order. */
__attribute__((target_clones("arch=skylake-avx512", "avx2", "default"), optimize("O3")))
static void q4k_block_dots(const uint8_t* qs, const int8_t* codes, int dot[8]) {
    for (uint32_t p = 0; p < 4; ++p) {
        int lo = 0, hi = 0;
        for (uint32_t k = 0; k < 32; ++k) {
            const uint8_t byte = qs[32 * p + k];
            lo += (int)codes[64 * p + k] * (int)(byte & 15);
            hi += (int)codes[64 * p + 32 + k] * (int)(byte >> 4);
        }
        dot[2 * p] = lo;
        dot[2 * p + 1] = hi;
    }
}

#if defined(__x86_64__)
#include <immintrin.h>
/* The same eight dots with the byte dot-product instruction where the host has it (unsigned nibbles x signed codes, four
 * products per 32-bit lane, no saturation: 4 x 15 x 127 fits): the form the reference's own AVX2 + VNNI rows take
 * (src/cpu/arch/avx2/routed_expert_avx2.cpp). Integer sums are exact in any order, so the bits do not change. */
__attribute__((target("avx2,avxvnni")))
static void q4k_block_dots_vnni(const uint8_t* qs, const int8_t* codes, int dot[8]) {
    const __m256i nibble = _mm256_set1_epi8(0x0f), zero = _mm256_setzero_si256();
    __m256i part[8];
    for (int p = 0; p < 4; ++p) {
        const __m256i q = _mm256_loadu_si256((const __m256i*)(qs + 32 * p));
        const __m256i lo = _mm256_and_si256(q, nibble), hi = _mm256_and_si256(_mm256_srli_epi16(q, 4), nibble);
        part[2 * p] = _mm256_dpbusd_avx_epi32(zero, lo, _mm256_loadu_si256((const __m256i*)(codes + 64 * p)));
        part[2 * p + 1] = _mm256_dpbusd_avx_epi32(zero, hi, _mm256_loadu_si256((const __m256i*)(codes + 64 * p + 32)));
    }
    /* eight vectors of eight partial sums -> one vector of the eight dots */
    const __m256i a = _mm256_hadd_epi32(_mm256_hadd_epi32(part[0], part[1]), _mm256_hadd_epi32(part[2], part[3]));
    const __m256i b = _mm256_hadd_epi32(_mm256_hadd_epi32(part[4], part[5]), _mm256_hadd_epi32(part[6], part[7]));
    const __m128i first = _mm_add_epi32(_mm256_castsi256_si128(a), _mm256_extracti128_si256(a, 1));
    const __m128i second = _mm_add_epi32(_mm256_castsi256_si128(b), _mm256_extracti128_si256(b, 1));
    _mm_storeu_si128((__m128i*)dot, first);
    _mm_storeu_si128((__m128i*)(dot + 4), second);
}
/* The whole row with the chain of the eight sub-blocks of a super-block in the eight lanes of a vector: every lane does the
 * scalar function's operations in the scalar function's order (products, one subtraction, the delta product; then x[2p] + x[2p+1]
 * and the pair accumulators), with separate multiplies and adds, so the bits are those of orc_q4k_row_a8's plain loop. */
__attribute__((target("avx2,avxvnni")))
static float q4k_row_a8_vnni(const uint8_t* wrow, uint32_t blocks, const int8_t* codes, const float* deltas, const int32_t* sums) {
    __m128 acc = _mm_setzero_ps();
    for (uint32_t b = 0; b < blocks; ++b) {
        const uint8_t* blk = wrow + (size_t)b * ORC_Q4_K_BLOCK;
        const float d = orc_half_to_float(le16(blk)), dm = orc_half_to_float(le16(blk + 2));
        int dots[8], sc[8], mn[8];
        q4k_block_dots_vnni(blk + 16, codes + 256 * b, dots);
        const uint32_t y = le32(blk + 4), z = le32(blk + 8), w = le32(blk + 12);
        for (unsigned j = 0; j < 4; ++j) {                      /* src/cpu/core/routed_expert.cpp:65-71 */
            const unsigned a8 = (y >> (8 * j)) & 255U, b8 = (z >> (8 * j)) & 255U, c8 = (w >> (8 * j)) & 255U;
            sc[j] = (int)(a8 & 63U); mn[j] = (int)(b8 & 63U);
            sc[4 + j] = (int)((c8 & 15U) | ((a8 >> 6U) << 4U)); mn[4 + j] = (int)((c8 >> 4U) | ((b8 >> 6U) << 4U));
        }
        const __m256 D = _mm256_mul_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(_mm256_loadu_si256((const __m256i*)sc)));
        const __m256 DM = _mm256_mul_ps(_mm256_set1_ps(dm), _mm256_cvtepi32_ps(_mm256_loadu_si256((const __m256i*)mn)));
        const __m256 u = _mm256_mul_ps(D, _mm256_cvtepi32_ps(_mm256_loadu_si256((const __m256i*)dots)));
        const __m256 v = _mm256_mul_ps(DM, _mm256_cvtepi32_ps(_mm256_loadu_si256((const __m256i*)(sums + 8 * b))));
        const __m256 x = _mm256_mul_ps(_mm256_loadu_ps(deltas + 8 * b), _mm256_sub_ps(u, v));
        const __m256 pairs = _mm256_hadd_ps(x, x);              /* x0+x1, x2+x3, (again) | x4+x5, x6+x7, (again) */
        const __m128 four = _mm_shuffle_ps(_mm256_castps256_ps128(pairs), _mm256_extractf128_ps(pairs, 1), _MM_SHUFFLE(1, 0, 1, 0));
        acc = _mm_add_ps(acc, four);
    }
    float a[4];
    _mm_storeu_ps(a, acc);
    const float s01 = a[0] + a[1], s23 = a[2] + a[3];
    return s01 + s23;
}
static int vector_rows_allowed = 1;
static int host_has_vnni(void) {
    static int known = -1;
    if (known < 0) known = __builtin_cpu_supports("avx2") && __builtin_cpu_supports("avxvnni") ? 1 : 0;
    return known && vector_rows_allowed;
}
#else
static float q4k_row_a8_vnni(const uint8_t* wrow, uint32_t blocks, const int8_t* codes, const float* deltas, const int32_t* sums) {
    (void)wrow; (void)blocks; (void)codes; (void)deltas; (void)sums;
    return 0.0F;
}
static int vector_rows_allowed = 1;
static int host_has_vnni(void) { return 0; }
#endif
/* Tests switch the vector form of the Q4_K row off to compare it with the plain loop; returns whether the host has it. */
int orc_vector_rows(int allowed) {
    vector_rows_allowed = allowed != 0;
    const int had = vector_rows_allowed;
    vector_rows_allowed = 1;
    const int has = host_has_vnni();
    vector_rows_allowed = had;
    return has;
}

float orc_q4k_row_a8(const uint8_t* wrow, uint32_t blocks, const int8_t* codes, const float* deltas,
                     const int32_t* sums) {
    if (host_has_vnni()) return q4k_row_a8_vnni(wrow, blocks, codes, deltas, sums);
    float acc[4] = {0.0F, 0.0F, 0.0F, 0.0F};
    for (uint32_t b = 0; b < blocks; ++b) {
        const uint8_t* blk = wrow + (size_t)b * ORC_Q4_K_BLOCK;
        const float d = orc_half_to_float(le16(blk)), dm = orc_half_to_float(le16(blk + 2));
        float x[8];
        int dots[8];
        q4k_block_dots(blk + 16, codes + 256 * b, dots);
        for (uint32_t j = 0; j < 8; ++j) {
            const int dot = dots[j];
            const float D = d * (float)orc_q4k_factor_words(blk, j, 0);
            const float DM = dm * (float)orc_q4k_factor_words(blk, j, 1);
            const float u = D * (float)dot;
            const float v = DM * (float)sums[8 * b + j];
            const float t = u - v;
            x[j] = deltas[8 * b + j] * t;
        }
        for (uint32_t p = 0; p < 4; ++p) acc[p] = acc[p] + (x[2 * p] + x[2 * p + 1]);
    }
    const float s01 = acc[0] + acc[1], s23 = acc[2] + acc[3];
    return s01 + s23;
}

/* src/cpu/core/routed_expert.cpp:73-108 with Q5K: 176-byte blocks (d, dmin, 12 factor bytes as in Q4_K, 32 fifth-bit bytes
 * - bit j of byte k belongs to element k of sub-block j -, 128 nibble bytes); q = nibble | fifth bit << 4. */
float orc_q5k_row_a8(const uint8_t* wrow, uint32_t blocks, const int8_t* codes, const float* deltas,
                     const int32_t* sums) {
    float acc[4] = {0.0F, 0.0F, 0.0F, 0.0F};
    for (uint32_t b = 0; b < blocks; ++b) {
        const uint8_t* blk = wrow + (size_t)b * ORC_Q5_K_BLOCK;
        const float d = orc_half_to_float(le16(blk)), dm = orc_half_to_float(le16(blk + 2));
        float x[8];
        for (uint32_t j = 0; j < 8; ++j) {
            const uint32_t p = j >> 1, hi = j & 1;
            int dot = 0;
            for (uint32_t k = 0; k < 32; ++k) {
                const uint8_t byte = blk[48 + 32 * p + k];
                int q = hi ? (byte >> 4) : (byte & 15);
                q |= ((blk[16 + k] >> j) & 1) << 4;
                dot += (int)codes[256 * b + 32 * j + k] * q;
            }
            const float D = d * (float)orc_q4k_factor_words(blk, j, 0);
            const float DM = dm * (float)orc_q4k_factor_words(blk, j, 1);
            const float u = D * (float)dot;
            const float v = DM * (float)sums[8 * b + j];
            const float t = u - v;
            x[j] = deltas[8 * b + j] * t;
        }
        for (uint32_t p = 0; p < 4; ++p) acc[p] = acc[p] + (x[2 * p] + x[2 * p + 1]);
    }
    const float s01 = acc[0] + acc[1], s23 = acc[2] + acc[3];
    return s01 + s23;
}

float orc_q4k_row_a8_contract_form(const uint8_t* wrow, uint32_t blocks, const int8_t* codes,
                                   const float* deltas, const int32_t* sums) {
    float acc[4] = {0.0F, 0.0F, 0.0F, 0.0F};
    for (uint32_t b = 0; b < blocks; ++b) {
        const uint8_t* blk = wrow + (size_t)b * ORC_Q4_K_BLOCK;
        const float d = orc_half_to_float(le16(blk)), dm = orc_half_to_float(le16(blk + 2));
        for (uint32_t pair = 0; pair < 4; ++pair) {
            float c[2];
            for (uint32_t h = 0; h < 2; ++h) {
                const uint32_t j = pair * 2 + h;
                uint8_t sc, mn;
                orc_q4k_scale_min(blk + 4, (int)j, &sc, &mn);
                int64_t raw = 0;
                for (uint32_t k = 0; k < 32; ++k) {
                    const uint8_t byte = blk[16 + (j / 2) * 32 + k];
                    raw += (int64_t)(j % 2 == 0 ? (byte & 15) : (byte >> 4)) * codes[256 * b + 32 * j + k];
                }
                const int32_t scaled = (int32_t)(raw * sc), minimum = sums[8 * b + j] * (int32_t)mn;
                const float u = d * (float)scaled;
                const float v = dm * (float)minimum;
                const float t = u - v;
                c[h] = deltas[8 * b + j] * t;
            }
            const float paired = c[0] + c[1];
            acc[pair] = acc[pair] + paired;
        }
    }
    const float left = acc[0] + acc[1], right = acc[2] + acc[3];
    return left + right;
}

float orc_q8_0_down_row_a8(const uint8_t* wrow, uint32_t groups, const int8_t* codes, const float* deltas) {
    float acc[4] = {0.0F, 0.0F, 0.0F, 0.0F};
    for (uint32_t g = 0; g < groups; ++g) {
        const uint8_t* blk = wrow + (size_t)g * ORC_Q8_0_BLOCK;
        const float d = orc_half_to_float(le16(blk));
        int dot = 0;
        for (uint32_t k = 0; k < 32; ++k) dot += (int)codes[32 * g + k] * (int)(int8_t)blk[2 + k];
        const float first = d * (float)dot;
        acc[g % 4] = acc[g % 4] + (deltas[g] * first);
    }
    const float s01 = acc[0] + acc[1], s23 = acc[2] + acc[3];
    return s01 + s23;
}

/* src/cpu/core/routed_expert.cpp:110-144 with Q51: block = fp16 d, fp16 m, 32 fifth bits, 16 nibble bytes; weight k is
 * nibble k % 16 (low halves for k < 16, high halves after) plus bit k of the fifth-bit word; the minimum enters through the
 * group's code sum. */
float orc_q5_1_down_row_a8(const uint8_t* wrow, uint32_t groups, const int8_t* codes, const float* deltas, const int32_t* sums) {
    float acc[4] = {0.0F, 0.0F, 0.0F, 0.0F};
    for (uint32_t g = 0; g < groups; ++g) {
        const uint8_t* blk = wrow + (size_t)g * ORC_Q5_1_BLOCK;
        const float d = orc_half_to_float(le16(blk)), m = orc_half_to_float(le16(blk + 2));
        const uint32_t fifth = (uint32_t)blk[4] | ((uint32_t)blk[5] << 8) | ((uint32_t)blk[6] << 16) | ((uint32_t)blk[7] << 24);
        int dot = 0;
        for (uint32_t k = 0; k < 32; ++k) {
            const uint8_t byte = blk[8 + (k & 15U)];
            const int q = (int)(k < 16 ? (byte & 15U) : (byte >> 4)) | (int)(((fifth >> k) & 1U) << 4);
            dot += (int)codes[32 * g + k] * q;
        }
        const float first = d * (float)dot;
        const float combined = first + (m * (float)sums[g]);
        acc[g % 4] = acc[g % 4] + (deltas[g] * combined);
    }
    const float s01 = acc[0] + acc[1], s23 = acc[2] + acc[3];
    return s01 + s23;
}

/* src/moe_a8_down_contract.cpp:18-37 (group term) and :147-158 (row): 210-byte blocks = 128 nibble bytes, 64 bytes of bit
 * pairs, 16 signed scales (one per 16 weights), fp16 d. */
float orc_q6k_down_row_a8(const uint8_t* wrow, uint32_t blocks, const int8_t* codes, const float* deltas) {
    float accum[4] = {0.0F, 0.0F, 0.0F, 0.0F};
    for (uint32_t block = 0; block < blocks; ++block) {
        const uint8_t* b = wrow + (size_t)block * ORC_Q6_K_BLOCK;
        const float d = orc_half_to_float(le16(b + 208));
        for (uint32_t pair = 0; pair < 4; ++pair) {
            float c[2];
            for (uint32_t k = 0; k < 2; ++k) {
                const uint32_t g = block * 8 + pair * 2 + k, j = g % 8, half = j / 4, quarter = j % 4;
                int64_t part[2] = {0, 0};
                for (uint32_t i = 0; i < 32; ++i) {
                    const uint32_t low = (b[half * 64 + (quarter & 1) * 32 + i] >> (quarter >= 2 ? 4 : 0)) & 15U;
                    const uint32_t high = (b[128 + half * 32 + i] >> (2 * quarter)) & 3U;
                    part[i / 16] += (int64_t)codes[g * 32 + i] * ((int)(low | (high << 4)) - 32);
                }
                const int64_t s0 = (int8_t)b[192 + 2 * j], s1 = (int8_t)b[193 + 2 * j];
                const int64_t integer = s0 * part[0] + s1 * part[1];
                c[k] = deltas[g] * (d * (float)integer);
            }
            const float paired = c[0] + c[1];
            accum[pair] = accum[pair] + paired;
        }
    }
    const float left = accum[0] + accum[1], right = accum[2] + accum[3];
    return left + right;
}

/* ------------------------------------------------------------------ exp / SwiGLU */
/* src/cpu/core/routed_expert.cpp:248-261 with v_exp = float(exp2(double(a))) (:212-216; the probe-table
 * corrections of :217-226 need tables that are not in the reference tree, so none apply here). */
float orc_expf_gfx1151(float x) {
    const float kLog2e = float_of(0x3fb8aa3bU), kLog2eLo = float_of(0x32a5705fU);
    const float ph = x * kLog2e;
    const float e = nearbyintf(ph);
    float pl = fmaf(x, kLog2e, -ph);
    pl = fmaf(x, kLog2eLo, pl);
    const float a = (ph - e) + pl;
    float y;
    if (fabsf(a) < 1.0F) y = scalbnf((float)exp2((double)a), (int)e);
    else y = a != a ? a : 0.0F;
    if (float_of(0xc2ce8ed0U) > x) y = 0.0F;
    if (float_of(0x42b17218U) < x) y = float_of(0x7f800000U);
    return y;
}

/* include/strix/ds41_moe.hpp:38-54 */
float orc_declared_exp(float x) {
    if (!(x == x)) return x;
    if (x > 88.0F) return float_of(0x7f800000U);
    if (x < -103.0F) return 0.0F;
    const float n = rintf(x * 1.44269504F);
    const float r = (x - n * 0.693359375F) - n * -2.12194440e-4F;
    float p = 1.98412698e-4F;
    p = p * r + 1.38888889e-3F;
    p = p * r + 8.33333333e-3F;
    p = p * r + 4.16666667e-2F;
    p = p * r + 1.66666667e-1F;
    p = p * r + 0.5F;
    p = p * r + 1.0F;
    p = p * r + 1.0F;
    const int k = (int)n, k1 = k / 2, k2 = k - k1;
    return (p * float_of((uint32_t)(k1 + 127) << 23)) * float_of((uint32_t)(k2 + 127) << 23);
}

static float exp_of(int kind, float x) {
    return kind == ORC_EXP_DECLARED ? orc_declared_exp(x) : kind == ORC_EXP_LIBM ? expf(x) : orc_expf_gfx1151(x);
}

int orc_swiglu_quantize(int exp_kind, const float* g, const float* u, int8_t* codes, float* delta, int32_t* sum,
                        float* h_out) {
    return orc_swiglu_quantize_clamped(exp_kind, INFINITY, g, u, codes, delta, sum, h_out);
}

int orc_swiglu_quantize_clamped(int exp_kind, float limit, const float* g, const float* u, int8_t* codes, float* delta,
                                int32_t* sum, float* h_out) {
    float hv[32];
    int bad = 0;
    for (int l = 0; l < 32; ++l) {
        /* include/strix/moe/activation_policy.hpp:22-24 */
        const float gc = g[l] > limit ? limit : g[l];
        const float uc = u[l] < -limit ? -limit : (u[l] > limit ? limit : u[l]);
        const float ex = exp_of(exp_kind, -gc);
        hv[l] = (gc / (1.0F + ex)) * uc;
        bad |= !is_finite(g[l]) || !is_finite(u[l]) || !is_finite(hv[l]);
    }
    if (h_out) for (int l = 0; l < 32; ++l) h_out[l] = hv[l];
    if (bad) return 0;
    float x = 0.0F;
    for (int l = 0; l < 32; ++l) x = fmaxf(x, fabsf(hv[l]));
    const int tiny = x > 0.0F && x < 0x1p-119F;
    const float dl = (x == 0.0F || tiny) ? 1.0F : x / 127.0F;
    int s = 0;
    for (int l = 0; l < 32; ++l) {
        const float rounded = tiny ? 0.0F : nearbyintf(hv[l] / dl);
        const int code = (int)fminf(127.0F, fmaxf(-127.0F, rounded));
        s += code;
        codes[l] = (int8_t)code;
    }
    *delta = dl;
    *sum = s;
    return 1;
}

/* ------------------------------------------------------------------ router */
void orc_route_select(const orc_route_policy* p, const float* scores, uint32_t* ids, float* weights) {
    /* include/strix/moe/route_policy.hpp:99-129, key float_serial, order selection, no selection bias. */
    uint8_t* taken = (uint8_t*)calloc(p->experts, 1);
    for (uint32_t k = 0; k < p->top_k; ++k) {
        uint32_t pick = p->experts;
        float best = 0.0F;
        for (uint32_t e = 0; e < p->experts; ++e) {
            if (taken[e]) continue;
            const float c = scores[e];
            if (pick == p->experts || c > best) { pick = e; best = c; }
        }
        taken[pick] = 1;
        ids[k] = pick;
    }
    free(taken);
    float sum = 0.0F;
    for (uint32_t k = 0; k < p->top_k; ++k) sum = sum + scores[ids[k]];
    const float denominator = sum + p->renorm_eps;
    for (uint32_t k = 0; k < p->top_k; ++k) {
        const float s = scores[ids[k]];
        const int renorm = p->renormalize && (p->top_k > 1U || p->renorm_single);
        weights[k] = (renorm ? s / denominator : s) * p->scale;
    }
}

void orc_route(const orc_route_policy* p, const float* x, uint32_t rows, uint32_t hidden, const float* w,
               const float* logit_bias, uint32_t* ids, float* weights, float* scores_out, float* logits_out,
               int threads) {
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(dynamic, 1)
    for (uint32_t r = 0; r < rows; ++r) {
        float* z = (float*)malloc(sizeof(float) * p->experts);
        float* s = (float*)malloc(sizeof(float) * p->experts);
        const float* xr = x + (size_t)r * hidden;
        for (uint32_t e = 0; e < p->experts; ++e) {
            const float* we = w + (size_t)e * hidden;
            float acc;
            if (p->logits_order == ORC_LOGITS_LANE32_BUTTERFLY) {      /* src/ds41_moe.cpp:74-83 */
                float lanes[32];
                for (int l = 0; l < 32; ++l) lanes[l] = 0.0F;
                for (uint32_t i = 0; i < hidden; ++i) lanes[i % 32] = lanes[i % 32] + we[i] * xr[i];
                acc = tree32(lanes);
            } else {                                                   /* tests/hip_moe_route_launcher_tests.hip:314-320 */
                acc = 0.0F;
                for (uint32_t i = 0; i < hidden; ++i) acc = fmaf(xr[i], we[i], acc);
            }
            z[e] = logit_bias ? acc + logit_bias[e] : acc;
        }
        /* include/strix/moe/route_policy.hpp:136-146 */
        float m = -INFINITY;
        for (uint32_t e = 0; e < p->experts; ++e) m = z[e] > m ? z[e] : m;
        float sum = 0.0F;
        for (uint32_t e = 0; e < p->experts; ++e) { s[e] = exp_of(p->exp_kind, z[e] - m); sum = sum + s[e]; }
        for (uint32_t e = 0; e < p->experts; ++e) s[e] = s[e] / sum;
        orc_route_select(p, s, ids + (size_t)r * p->top_k, weights + (size_t)r * p->top_k);
        if (scores_out) memcpy(scores_out + (size_t)r * p->experts, s, sizeof(float) * p->experts);
        if (logits_out) memcpy(logits_out + (size_t)r * p->experts, z, sizeof(float) * p->experts);
        free(z); free(s);
    }
}

/* ------------------------------------------------------------------ combine */
/* include/strix/moe/combine.hpp:24-33: nearest-even into the upper 16 bits; a NaN is returned as it came */
static float combine_round_bf16(float x) {
    uint32_t bits;
    memcpy(&bits, &x, 4);
    if ((bits & 0x7f800000U) == 0x7f800000U && (bits & 0x7fffffU)) return x;
    bits = (bits + 0x7fffU + ((bits >> 16) & 1U)) & 0xffff0000U;
    memcpy(&x, &bits, 4);
    return x;
}

void orc_combine(int form, uint32_t rows, uint32_t top_k, uint32_t width, const float* w, const uint32_t* ids,
                 const float* raw, const float* base, float* y) {
    if (form == ORC_COMBINE_BF16_STEPS || form == ORC_COMBINE_BF16_STEPS_ROUNDED_EO) {
        for (uint32_t r = 0; r < rows; ++r)
            for (uint32_t d = 0; d < width; ++d) {
                float acc = 0.0F;
                for (uint32_t k = 0; k < top_k; ++k) {
                    float e = raw[((size_t)r * top_k + k) * width + d];
                    if (form == ORC_COMBINE_BF16_STEPS_ROUNDED_EO) e = combine_round_bf16(e);   /* route_wave_kernel.hpp:113-114 */
                    const float term = w ? combine_round_bf16(e * w[(size_t)r * top_k + k]) : e;  /* combine.hpp:52 */
                    acc = combine_round_bf16(acc + term);                                         /* combine.hpp:53 */
                }
                const size_t at = (size_t)r * width + d;
                y[at] = base ? combine_round_bf16(acc + base[at]) : acc;                          /* combine.hpp:57 */
            }
        return;
    }
    for (uint32_t r = 0; r < rows; ++r) {
        uint32_t order[64];
        for (uint32_t k = 0; k < top_k; ++k) order[k] = k;
        if (form == ORC_COMBINE_MULADD_ASCENDING_EXPERT)     /* src/ds41_moe.cpp:26-31: slots by ascending expert id */
            for (uint32_t i = 1; i < top_k; ++i)
                for (uint32_t j = i; j > 0 && ids[(size_t)r * top_k + order[j]] < ids[(size_t)r * top_k + order[j - 1]]; --j) {
                    const uint32_t t = order[j]; order[j] = order[j - 1]; order[j - 1] = t;
                }
        for (uint32_t d = 0; d < width; ++d) {
            float acc = 0.0F;
            for (uint32_t k = 0; k < top_k; ++k) {
                const uint32_t slot = order[k];
                const float e = raw[((size_t)r * top_k + slot) * width + d];
                const float wk = w[(size_t)r * top_k + slot];
                if (form == ORC_COMBINE_FMA_SLOT_ORDER) acc = fmaf(wk, e, acc);   /* include/strix/moe/combine.hpp:50 */
                else acc = acc + wk * e;                                          /* src/ds41_expert_tp.cpp:193-197 */
            }
            const size_t at = (size_t)r * width + d;
            y[at] = base ? acc + base[at] : acc;
        }
    }
}

void orc_combine_shared(int form, uint32_t rows, uint32_t top_k, uint32_t shared_slots, uint32_t width, const float* w, const uint32_t* ids,
                        const float* raw, const float* base, float* y) {
    const uint32_t routed = top_k - shared_slots;
    for (uint32_t r = 0; r < rows; ++r) {
        /* the routed slots in the form's order (the always-on ids are the largest, so they are last in both orders) */
        orc_combine(form, 1, routed, width, w + (size_t)r * top_k, ids + (size_t)r * top_k, raw + (size_t)r * top_k * width, NULL, y + (size_t)r * width);
        for (uint32_t d = 0; d < width; ++d) {
            float acc = y[(size_t)r * width + d];
            for (uint32_t k = routed; k < top_k; ++k) {
                const float product = w[(size_t)r * top_k + k] * raw[((size_t)r * top_k + k) * width + d];
                acc = acc + product;
            }
            y[(size_t)r * width + d] = base ? acc + base[(size_t)r * width + d] : acc;
        }
    }
}

void orc_dense_a8_quantize(const float* x, uint32_t width, int8_t* codes, float* deltas) {
    for (uint32_t g = 0; g < width / 32; ++g) {                 /* src/hip_q8_rows_gemv.hpp:1232-1250 */
        int bad = 0;
        float amax = 0.0F;
        for (uint32_t k = 0; k < 32; ++k) {
            const float v = x[g * 32 + k];
            bad |= !isfinite(v);
            amax = fmaxf(amax, fabsf(v));
        }
        const int tiny = amax > 0.0F && amax < 0x1p-119F;
        uint32_t nan_bits = 0x7fc00000U;
        float nan_value;
        memcpy(&nan_value, &nan_bits, 4);
        const float delta = bad ? nan_value : (amax == 0.0F || tiny) ? 1.0F : amax / 127.0F;
        deltas[g] = delta;
        for (uint32_t k = 0; k < 32; ++k) {
            const float rounded = (bad || tiny) ? 0.0F : rintf(x[g * 32 + k] / delta);
            codes[g * 32 + k] = (int8_t)(int)fminf(127.0F, fmaxf(-127.0F, rounded));
        }
    }
}

void orc_gemv_q8_0_a8_chain(const uint8_t* weight, uint32_t row_bytes, const int8_t* codes, const float* deltas, uint32_t in, uint32_t count,
                            uint32_t rows, uint32_t x_stride, float* out, uint32_t out_stride) {
    for (uint32_t r = 0; r < rows; ++r)
        for (uint32_t o = 0; o < count; ++o) {
            float acc = 0.0F;
            for (uint32_t b = 0; b < in / 32; ++b) {            /* src/hip_q8_rows_gemv.hpp:1162-1165 */
                const uint8_t* p = weight + (size_t)o * row_bytes + (size_t)b * 34;
                int32_t dot = 0;
                for (uint32_t k = 0; k < 32; ++k) dot += (int32_t)(int8_t)p[2 + k] * (int32_t)codes[(size_t)r * x_stride + b * 32 + k];
                const float scale = orc_half_to_float((uint16_t)(p[0] | (p[1] << 8))) * deltas[(size_t)r * (x_stride / 32) + b];
                acc = fmaf(scale, (float)dot, acc);
            }
            if (isnan(acc)) { const uint32_t bits = 0x7fc00000U; memcpy(&acc, &bits, 4); }
            out[(size_t)r * out_stride + o] = acc;
        }
}

void orc_shared_gate(const float* x, const float* w, uint32_t rows, uint32_t hidden, int exp_kind, float* gate, float* dots) {
    for (uint32_t r = 0; r < rows; ++r) {
        float s[256];
        for (uint32_t t = 0; t < 256; ++t) {                  /* src/hip_shared_expert_launcher.hip:629-632 */
            float sum = 0.0F;
            for (uint32_t f = t; f < hidden; f += 256) sum = fmaf(x[(size_t)r * hidden + f], w[f], sum);
            s[t] = sum;
        }
        for (uint32_t h = 128; h >= 1; h >>= 1)                /* src/core/ordered_reduce.hpp:8-9 */
            for (uint32_t l = 0; l < h; ++l) s[l] = s[l] + s[l + h];
        if (dots) dots[r] = s[0];
        gate[r] = 1.0F / (1.0F + exp_of(exp_kind, -s[0]));      /* :635 */
    }
}

/* ------------------------------------------------------------------ routed experts */
static const uint8_t* gate_row_ptr(const orc_expert_weights* w, const uint8_t* base, uint32_t expert, uint32_t o) {
    return base + (size_t)expert * w->gate_expert_stride + (size_t)o * w->gate_row_stride;
}

void orc_routed_down(const orc_expert_weights* w, const orc_expert_job* job, int threads) {
    const uint32_t hidden = w->hidden, ffn = w->ffn, groups = ffn / 32, n = job->rows * w->top_k;
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(dynamic, 64) collapse(2)
    for (uint32_t a = 0; a < n; ++a)
        for (uint32_t o = 0; o < hidden; ++o) {
            const uint32_t expert = job->ids[a];
            const uint8_t* wrow = w->down + (size_t)expert * w->down_expert_stride + (size_t)o * w->down_row_stride;
            const int8_t* c = job->h_codes + (size_t)a * ffn;
            const float* d = job->h_deltas + (size_t)a * groups;
            const int32_t* s = job->h_sums + (size_t)a * groups;
            float value;
            if (w->down_type == ORC_Q4_K) value = orc_q4k_row_a8(wrow, ffn / 256, c, d, s);   /* src/moe_a8_down_contract.cpp:146 */
            else if (w->down_type == ORC_Q5_1) value = orc_q5_1_down_row_a8(wrow, groups, c, d, s);
            else if (w->down_type == ORC_Q6_K) value = orc_q6k_down_row_a8(wrow, ffn / 256, c, d);
            else value = orc_q8_0_down_row_a8(wrow, groups, c, d);
            job->rawdots[(size_t)a * hidden + o] = value;
        }
}

int orc_routed_experts(const orc_expert_weights* w, const orc_expert_job* job, int threads) {
    const uint32_t hidden = w->hidden, ffn = w->ffn, blocks = hidden / 256, groups = ffn / 32;
    const uint32_t n = job->rows * w->top_k;
    int8_t* hc = job->h_codes ? job->h_codes : (int8_t*)malloc((size_t)n * ffn);
    float* hd = job->h_deltas ? job->h_deltas : (float*)malloc(sizeof(float) * (size_t)n * groups);
    int32_t* hs = job->h_sums ? job->h_sums : (int32_t*)malloc(sizeof(int32_t) * (size_t)n * groups);
    int bad = 0;
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(dynamic, 1) collapse(2) reduction(| : bad)
    for (uint32_t a = 0; a < n; ++a)
        for (uint32_t grp = 0; grp < groups; ++grp) {
            const uint32_t row = a / w->top_k, expert = job->ids[a];
            const int8_t* codes = job->codes + (size_t)row * hidden;
            const float* deltas = job->deltas + (size_t)row * (hidden / 32);
            const int32_t* sums = job->sums + (size_t)row * (hidden / 32);
            float g[32], u[32], h[32];
            for (uint32_t l = 0; l < 32; ++l) {
                const uint32_t o = grp * 32 + l;
                if (w->gate_type == ORC_Q5_K) {
                    g[l] = orc_q5k_row_a8(gate_row_ptr(w, w->gate, expert, o), blocks, codes, deltas, sums);
                    u[l] = orc_q5k_row_a8(gate_row_ptr(w, w->up, expert, o), blocks, codes, deltas, sums);
                } else {
                    g[l] = orc_q4k_row_a8(gate_row_ptr(w, w->gate, expert, o), blocks, codes, deltas, sums);
                    u[l] = orc_q4k_row_a8(gate_row_ptr(w, w->up, expert, o), blocks, codes, deltas, sums);
                }
            }
            if (job->gate_out) memcpy(job->gate_out + (size_t)a * ffn + grp * 32, g, sizeof g);
            if (job->up_out) memcpy(job->up_out + (size_t)a * ffn + grp * 32, u, sizeof u);
            const int ok = orc_swiglu_quantize_clamped(w->exp_kind, w->swiglu_limit == 0.0F ? INFINITY : w->swiglu_limit, g, u, hc + (size_t)a * ffn + grp * 32,
                                               hd + (size_t)a * groups + grp, hs + (size_t)a * groups + grp, h);
            if (job->h_out) memcpy(job->h_out + (size_t)a * ffn + grp * 32, h, sizeof h);
            if (!ok) {
                bad |= 1;
                if (job->status) {
#pragma omp atomic
                    job->status[row] |= ORC_STATUS_NONFINITE_PROJECTION;
                }
            }
        }
    if (!bad) {
        orc_expert_job down = *job;
        down.h_codes = hc; down.h_deltas = hd; down.h_sums = hs;
        orc_routed_down(w, &down, threads);
    }
    if (!job->h_codes) free(hc);
    if (!job->h_deltas) free(hd);
    if (!job->h_sums) free(hs);
    return bad;
}

/* ------------------------------------------------------------------ BASE class */
float orc_lane_dot(const float* a, const float* b, size_t n) {   /* include/strix/ds41_layer.hpp:96-108 */
    float v[32];
    for (int l = 0; l < 32; ++l) v[l] = 0.0F;
    for (size_t l = 0; l < 32; ++l)
        for (size_t i = l; i < n; i += 32) v[l] = v[l] + a[i] * b[i];
    return tree32(v);
}

void orc_base_linear(uint32_t type, const uint8_t* weight, uint64_t row_stride, uint32_t outputs, uint32_t in,
                     const float* x, uint32_t rows, uint32_t x_stride, float* y, uint32_t y_stride, int threads) {
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
    for (uint32_t o = 0; o < outputs; ++o) {
        float* wr = (float*)malloc(sizeof(float) * in);
        if (type == ORC_Q4_K) orc_dequant_q4_k_row(weight + (size_t)o * row_stride, in, wr);
        else orc_dequant_q8_0_row(weight + (size_t)o * row_stride, in, wr);
        for (uint32_t r = 0; r < rows; ++r) {
            double acc = 0.0;
            const float* xr = x + (size_t)r * x_stride;
            for (uint32_t k = 0; k < in; ++k) acc += (double)wr[k] * (double)xr[k];
            y[(size_t)r * y_stride + o] = (float)acc;
        }
        free(wr);
    }
}
