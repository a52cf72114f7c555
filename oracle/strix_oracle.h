/*
 * TEST INFRASTRUCTURE - the CPU parity oracle. Not part of the shipped library.
 *
 * A plain-C restatement of the reference's CPU arithmetic for the quantized weight-product path
 * (Q8_0 / Q4_K block decode, the A8 int8-activation contract, Q8_0xA8 and Q4_KxA8 products, SwiGLU +
 * re-quantisation, softmax router policy, ordered combine, expert tensor-parallel rank partials, and
 * the exact-weight "BASE" products used to judge the fp16 prefill form). Only tests, the smoke check
 * and the cpu_baseline leg of the benchmark may load it; the GPU library never links or calls it.
 *
 * Every function names the reference file:line it restates. Compile with -ffp-contract=off and
 * without fast-math: every float operation below is one IEEE-754 binary32 round-to-nearest operation.
 *
 * Pinning status (what checks each function besides this text):
 *   half/Q8_0/Q4_K decode, scale/min unpack, Q8_0 writer, A8 quantiser, RMSNorm, Q8_0xA8 product order,
 *   Q4_KxA8 and Q5_KxA8 rows, Q8_0, Q5_1 and Q6_K down rows, router selection/weights, combine: pinned by the literal vectors and
 *   invariants of the reference's own tests (tests/golden/) and, where it builds, bitwise against the
 *   compiled reference (oracle/_ref).
 *   orc_expf_gfx1151: pinned only against the reference function run with EMPTY correction tables;
 *   the real gfx1151 probe tables are not in the reference tree -> parity with gfx1151 hardware
 *   exp is UNPINNED.
 *   orc_quantize_q4_k_row (fp32 -> Q4_K writer): the reference has no such writer -> parity unpinned
 *   (any valid writer serves: parity is defined from the packed bytes onward).
 *   Expert tensor-parallel rank partial on Q4_K blocks (orc_routed_experts with the rank's ffn share and the
 *   full-matrix strides, then orc_combine in the mul-then-add ascending-expert form): the reference declares the
 *   split for its own TP pack only; the Q4_K form here keeps its structure (rank-local SwiGLU groups, rank-local
 *   K blocks, fold in ascending expert id) -> pinned by invariants only, parity unpinned.
 */
#ifndef STRIX_ORACLE_H
#define STRIX_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORC_Q5_1 = 7, ORC_Q8_0 = 8, ORC_Q4_K = 12, ORC_Q5_K = 13, ORC_Q6_K = 14 };          /* ggml type ids */
enum { ORC_Q5_1_BLOCK = 24, ORC_Q8_0_BLOCK = 34, ORC_Q4_K_BLOCK = 144, ORC_Q5_K_BLOCK = 176, ORC_Q6_K_BLOCK = 210 };
enum { ORC_STATUS_INVALID_ROUTE = 1, ORC_STATUS_NONFINITE_ACTIVATION = 2, ORC_STATUS_INVALID_DELTA = 4,
       ORC_STATUS_NONFINITE_PROJECTION = 8 };
enum { ORC_EXP_GFX1151_NOTABLE = 0, ORC_EXP_DECLARED = 1,
       ORC_EXP_LIBM = 2 };   /* expf of the C library: the Math::exp of the reference's router test oracle (tests/hip_moe_route_launcher_tests.hip:329) */
enum { ORC_LOGITS_FMA_ASCENDING = 0, ORC_LOGITS_LANE32_BUTTERFLY = 1 };
enum { ORC_COMBINE_FMA_SLOT_ORDER = 0, ORC_COMBINE_MULADD_ASCENDING_EXPERT = 1, ORC_COMBINE_BF16_STEPS = 3,
       ORC_COMBINE_BF16_STEPS_ROUNDED_EO = 4 };

/* ---- scalar conversions --------------------------------------------------------------------- */
float orc_half_to_float(uint16_t bits);        /* src/cpu/core/reference.cpp:15-24 */
uint16_t orc_float_to_half(float value);       /* IEEE round-to-nearest-even narrowing (writer side only) */

/* ---- block decode (bitwise llama.cpp order) -------------------------------------------------- */
void orc_dequant_q8_0_row(const uint8_t* row, size_t elements, float* out);   /* src/ggml_dequant.cpp:84-87 */
void orc_dequant_q4_k_row(const uint8_t* row, size_t elements, float* out);   /* src/ggml_dequant.cpp:119-130 */
/* 6-bit scale/min of sub-block j, byte formulation (src/ggml_dequant.cpp:43-50). */
void orc_q4k_scale_min(const uint8_t* scales12, int j, uint8_t* scale, uint8_t* minimum);
/* Same factors, 32-bit word formulation (src/cpu/core/routed_expert.cpp:65-71). */
unsigned orc_q4k_factor_words(const uint8_t* block144, unsigned group, int minimum);

/* ---- writers (build test weights) ------------------------------------------------------------ */
void orc_quantize_q8_0_row(const float* x, size_t elements, uint8_t* out);    /* include/strix/q8_0_rule.hpp:25-33 */
void orc_quantize_q4_k_row(const float* x, size_t elements, uint8_t* out);    /* no reference counterpart */

/* ---- A8 activation quantiser ----------------------------------------------------------------- */
/* tiny_rule != 0: src/cpu/core/reference.cpp:35-55 (amax < 2^-119 -> delta 1, codes 0).
 * tiny_rule == 0: src/moe_q4k_a8_contract.cpp:67-96. Returns 0, or -1 when width % 32 != 0 (nothing written).
 * Returns 1 when a value is non-finite (contract form rejects it; outputs then unspecified). sums may be NULL. */
int orc_quantize_a8(const float* x, size_t width, int8_t* codes, float* deltas, int32_t* sums, int tiny_rule);

/* ---- Q8_0 x A8 dense product (src/cpu/core/reference.cpp:57-84, src/core/integer_math.hpp:11-13,43-47) */
typedef struct {
    const uint8_t* weight;   /* output o at weight + o * row_bytes */
    const int8_t* codes;     /* row r at codes + r * x_stride */
    const float* deltas;     /* deltas[r * (x_stride / 32) + k / 32] */
    float* out;              /* out[r * out_stride + o] */
    uint32_t row_bytes, in, count, rows, x_stride, out_stride;
    uint32_t accumulate;
} orc_q8a8_view;
int orc_gemv_q8_0_a8(const orc_q8a8_view* view, int threads);   /* -1: in % 32 != 0, nothing written */

/* ---- Q4_K x A8 row (src/cpu/core/routed_expert.cpp:73-108 == src/moe_q4k_a8_contract.cpp:126-140) */
void orc_rmsnorm_f32(const float* x, const float* w, uint32_t n, float eps, float* y, uint32_t rows);
/* The Q4_K row has a vector form (byte dot-product instruction, the chain of a super-block's eight sub-blocks in eight
 * lanes) on hosts with AVX2 + AVX-VNNI; same operations in the same order, same bits. orc_vector_rows(0) makes every later
 * call take the plain loop, orc_vector_rows(1) allows the vector form again; returns 1 when the host has the vector form. */
int orc_vector_rows(int allowed);
float orc_q4k_row_a8(const uint8_t* wrow, uint32_t blocks, const int8_t* codes, const float* deltas,
                     const int32_t* sums);
float orc_q5k_row_a8(const uint8_t* wrow, uint32_t blocks, const int8_t* codes, const float* deltas,
                     const int32_t* sums);
/* The contract's formulation d * float(scale * dot) (src/moe_q4k_a8_contract.cpp:40-58). Same bits. */
float orc_q4k_row_a8_contract_form(const uint8_t* wrow, uint32_t blocks, const int8_t* codes,
                                   const float* deltas, const int32_t* sums);
/* Q8_0 down row, groups mod 4 (src/cpu/core/routed_expert.cpp:110-144 with Q51 = false). */
float orc_q8_0_down_row_a8(const uint8_t* wrow, uint32_t groups, const int8_t* codes, const float* deltas);
float orc_q6k_down_row_a8(const uint8_t* wrow, uint32_t blocks, const int8_t* codes, const float* deltas);
float orc_q5_1_down_row_a8(const uint8_t* wrow, uint32_t groups, const int8_t* codes, const float* deltas, const int32_t* sums);

/* ---- exp / SwiGLU ---------------------------------------------------------------------------- */
float orc_expf_gfx1151(float x);     /* src/cpu/core/routed_expert.cpp:212-261 with empty tables */
float orc_declared_exp(float x);     /* include/strix/ds41_moe.hpp:38-54 */
/* h = (g / (1 + exp(-g))) * u over one 32-output group, then A8 with the tiny rule.
 * Returns 1 and writes codes/delta/sum, or 0 (writes nothing) when g, u or h is non-finite.
 * h_out (optional) receives the 32 h values. src/cpu/core/routed_expert.cpp:147-170. */
int orc_swiglu_quantize(int exp_kind, const float* g, const float* u, int8_t* codes, float* delta,
                        int32_t* sum, float* h_out);
/* The same with the SwiGLU clamp trait (include/strix/moe/activation_policy.hpp:22-24; producer body
 * src/hip_moe_q4k_a8_probe.hip:594-621): g = min(g, limit), u = clamp(u, -limit, limit) before silu(g) * u, the finite check
 * stays on the raw g and u. limit = +infinity clamps nothing. */
int orc_swiglu_quantize_clamped(int exp_kind, float limit, const float* g, const float* u, int8_t* codes, float* delta,
                                int32_t* sum, float* h_out);

/* ---- router (include/strix/moe/route_policy.hpp:99-156; logits tests/hip_moe_route_launcher_tests.hip:281-330) */
typedef struct {
    uint32_t experts, top_k;
    int logits_order;       /* ORC_LOGITS_* */
    int exp_kind;           /* Math::exp of the softmax */
    float renorm_eps;       /* Qwen launcher 0, policy default 1e-20 */
    float scale;
    int renormalize;
    int renorm_single;      /* renormalise when renormalize && (top_k > 1 || renorm_single), include/strix/moe/route_policy.hpp:146 */
} orc_route_policy;
/* x [rows][hidden] fp32, w [experts][hidden] fp32, logit_bias [experts] or NULL (added to the logit).
 * ids/weights [rows][top_k]; scores (optional) [rows][experts]; logits (optional) [rows][experts]. */
void orc_route(const orc_route_policy* p, const float* x, uint32_t rows, uint32_t hidden, const float* w,
               const float* logit_bias, uint32_t* ids, float* weights, float* scores, float* logits, int threads);
/* Selection + weights only from given scores (route_select_ref, float_serial key, selection order). */
void orc_route_select(const orc_route_policy* p, const float* scores, uint32_t* ids, float* weights);

/* ---- combine (include/strix/moe/combine.hpp:36-59; src/ds41_expert_tp.cpp:189-199) ------------- */
/* raw [rows][top_k][width], w [rows][top_k], ids [rows][top_k] (needed for the ascending-expert form),
 * base [rows][width] or NULL, y [rows][width]. The bf16-steps forms (combine.hpp:52-57; operands rounded on read:
 * src/moe_core/route_wave_kernel.hpp:112-120) take w == NULL as unit weights and round every step to bfloat16. */
void orc_combine(int form, uint32_t rows, uint32_t top_k, uint32_t width, const float* w, const uint32_t* ids,
                 const float* raw, const float* base, float* y);

/* The ordered combine of a layer whose last `shared_slots` slots are always-on experts: those enter as acc + (w * value), product
 * and sum rounded separately, in both forms (the gate scales the shared expert's output with one multiply,
 * src/hip_shared_expert_launcher.hip:727,779; the sum with the routed row is one add, include/strix/moe/combine.hpp:56). */
void orc_combine_shared(int form, uint32_t rows, uint32_t top_k, uint32_t shared_slots, uint32_t width, const float* w, const uint32_t* ids,
                        const float* raw, const float* base, float* y);

/* ---- the dense A8 profile of the reference's Q8_0 projections (src/hip_q8_rows_gemv.hpp:1155-1170,1232-1250; host statement of the
 * row contract: tests/dense_a8_small_reference_tests.cpp:93-104)
 * quantiser, per block of 32: any non-finite x -> delta = NaN (0x7fc00000), codes 0; tiny = 0 < amax < 2^-119; delta = (amax == 0 ||
 * tiny) ? 1 : amax / 127; code = tiny ? 0 : clamp(rint(x / delta), -127, 127).
 * product: acc = +0; acc = fma(float(d_w) * delta, float(dot), acc) over the blocks in ascending order; a NaN result is 0x7fc00000.
 * Parity: device code only in the reference (no compiled form here); pinned by order fixtures that the tree32 order of
 * orc_gemv_q8_0_a8, an unfused multiply-add or the other association of the three-factor product changes. */
void orc_dense_a8_quantize(const float* x, uint32_t width, int8_t* codes, float* deltas);
void orc_gemv_q8_0_a8_chain(const uint8_t* weight, uint32_t row_bytes, const int8_t* codes, const float* deltas, uint32_t in, uint32_t count,
                            uint32_t rows, uint32_t x_stride, float* out, uint32_t out_stride);

/* ---- the shared expert's scalar gate (src/hip_shared_expert_launcher.hip:624-645 shared_gate_dot; tree src/core/ordered_reduce.hpp:8-16)
 * x [rows][hidden] fp32 values of the stored activations, w [hidden]; gate [rows] = 1 / (1 + exp(-dot)):
 * 256 thread-strided fma chains (thread t: features t, t + 256, ... ascending; the reference's build fuses `sum += x * w`, its
 * target sets no contraction flag), halving tree s[l] = s[l] + s[l + h] for h = 128 .. 1, exp of the given kind, one division.
 * Parity: the device header cannot be compiled into oracle/_ref; pinned by order fixtures (tests/test_oracle_golden.py) that a
 * sequential or adjacent-pair reduction, or an unfused multiply-add, changes. dots: optional [rows], the value before the sigmoid. */
void orc_shared_gate(const float* x, const float* w, uint32_t rows, uint32_t hidden, int exp_kind, float* gate, float* dots);

/* ---- routed expert layer (src/cpu/core/routed_expert.cpp:264-300 generalised to Q4_K / Q8_0 down) - */
typedef struct {
    uint32_t hidden, ffn, experts, top_k;   /* ffn = intermediate rows computed here (rank-local for a TP shard) */
    uint32_t gate_type, down_type;          /* ORC_Q4_K or ORC_Q5_K gate/up; ORC_Q4_K, ORC_Q8_0, ORC_Q5_1 or ORC_Q6_K down */
    const uint8_t *gate, *up, *down;
    uint64_t gate_expert_stride, gate_row_stride;   /* bytes */
    uint64_t down_expert_stride, down_row_stride;   /* bytes; a rank reads the first ffn/blk blocks of each row */
    int exp_kind;
    float swiglu_limit;     /* clamp trait; +infinity or 0 = none */
} orc_expert_weights;
typedef struct {
    /* inputs */
    const int8_t* codes; const float* deltas; const int32_t* sums;   /* [rows][hidden], [rows][hidden/32] x2 */
    const uint32_t* ids;                                             /* [rows][top_k] */
    uint32_t rows;
    /* outputs (any may be NULL except rawdots) */
    float* gate_out;      /* [rows][top_k][ffn] */
    float* up_out;        /* [rows][top_k][ffn] */
    float* h_out;         /* [rows][top_k][ffn] */
    int8_t* h_codes;      /* [rows][top_k][ffn] */
    float* h_deltas;      /* [rows][top_k][ffn/32] */
    int32_t* h_sums;      /* [rows][top_k][ffn/32] */
    float* rawdots;       /* [rows][top_k][hidden] */
    uint32_t* status;     /* [rows], OR-ed */
} orc_expert_job;
/* Returns 0, or 1 when a non-finite projection stopped the job before the down phase (rawdots untouched). */
int orc_routed_experts(const orc_expert_weights* w, const orc_expert_job* job, int threads);
/* Down phase alone from a given h image (stage-by-stage parity with device-provided intermediates). */
void orc_routed_down(const orc_expert_weights* w, const orc_expert_job* job, int threads);

/* ---- BASE class: exact dequantised weights x fp32 activations ------------------------------------ */
/* y[r][o] = sum_k double(dequant(W[o][k])) * double(x[r][k]), rounded once to fp32. */
void orc_base_linear(uint32_t type, const uint8_t* weight, uint64_t row_stride, uint32_t outputs, uint32_t in,
                     const float* x, uint32_t rows, uint32_t x_stride, float* y, uint32_t y_stride, int threads);
/* Lane-32 strided dot + butterfly in fp32 (include/strix/ds41_layer.hpp:96-108). */
float orc_lane_dot(const float* a, const float* b, size_t n);

int orc_max_threads(void);
/* seconds for `reps` multi-thread read passes over a buffer of 64-bit words (host memory-read ceiling) */
double orc_read_seconds(const uint64_t* buffer, size_t words, int reps, int threads, uint64_t* checksum);

#ifdef __cplusplus
}
#endif
#endif
