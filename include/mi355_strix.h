/*
 * mi355_strix.h - C ABI of the MI355X (gfx950) implementation of the engine's quantized weight-product path:
 * GGUF Q8_0 / Q4_K decode products on int8 ("A8") activations, the softmax MoE router, the expert-grouped
 * SwiGLU gate/up/down products with the ordered combine, and one rank's partial sums of the expert
 * tensor-parallel split. Plain pointers and sizes only; every pointer is DEVICE memory unless said otherwise.
 *
 * Conventions (those of the reference's enqueue_* entry points, include/strix/hip_moe_q4k_a8_probe.hpp:8-11):
 *   - an entry point validates its arguments on the host, then only enqueues kernels on `stream`; it never
 *     allocates, synchronises, resets or reads back. The caller owns every buffer until the stream is idle.
 *   - return value: 0 on success; a negative MI355_E_* on an admission failure (nothing was enqueued and no
 *     buffer was written; mi355_last_error() holds the reason for the calling thread). Nothing throws.
 *   - numerical problems are reported on the device, in the caller's sticky per-row status words
 *     (bits below = include/strix/hip_moe_q4k_a8_probe.hpp:7, include/strix/moe_a8_down_contract.hpp:53-54).
 *   - arithmetic: the reference's A8 class. Every product is an exact int32 group dot followed by the
 *     declared chain of single-rounding fp32 operations (no contraction), so gate/up/down values and the
 *     combine are bitwise those of the reference CPU functions named at each entry point.
 */
#ifndef MI355_STRIX_H
#define MI355_STRIX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* mi355_stream;   /* hipStream_t */

enum {
    MI355_OK = 0,
    MI355_E_INVALID_ARGUMENT = -1,   /* shape / alignment / null pointer: std::invalid_argument in the reference */
    MI355_E_UNSUPPORTED = -2,        /* a weight type or form this library does not implement */
    MI355_E_HIP = -3,                /* a HIP runtime call failed (hip_check in the reference) */
    MI355_E_NO_DEVICE = -4
};

/* device status word bits */
enum {
    MI355_STATUS_INVALID_ROUTE = 1,          /* route id >= experts, or non-finite route weight */
    MI355_STATUS_NONFINITE_ACTIVATION = 2,   /* non-finite input activation */
    MI355_STATUS_INVALID_DELTA = 4,
    MI355_STATUS_NONFINITE_PROJECTION = 8,   /* non-finite gate, up or h (the fp16 prefill form: h beyond fp16 too); the down
                                                phase of the job is skipped and its merge publishes no row */
    MI355_STATUS_AGGREGATE = 16              /* merged output failed the commit threshold */
};

enum { MI355_TYPE_Q5_1 = 7, MI355_TYPE_Q8_0 = 8, MI355_TYPE_Q4_K = 12, MI355_TYPE_Q5_K = 13, MI355_TYPE_Q6_K = 14 };              /* ggml tensor type ids */
enum { MI355_INPUT_F32 = 0, MI355_INPUT_F16 = 1, MI355_INPUT_BF16 = 2 };
enum { MI355_LOGITS_FMA_ASCENDING = 0, MI355_LOGITS_LANE32_BUTTERFLY = 1 };
enum { MI355_COMBINE_FMA_SLOT_ORDER = 0, MI355_COMBINE_MULADD_ASCENDING_EXPERT = 1,
       MI355_COMBINE_BF16_STEPS = 3,   /* mi355_moe_enqueue_combine only: every step of the reduction rounded to bfloat16 */
       MI355_COMBINE_NONE = 2 };   /* mi355_moe_enqueue_prefill_f16 only: stop after the down rows. rawdots then holds the unweighted
                                      per-slot outputs; for a top-1 layer of weight 1 (an always-on shared expert) rawdots[row] is
                                      the layer's output - fma(1, x, 0) = x - and can be the `base` of the routed call, which saves
                                      the copy a combine of one slot would be. The caller reads status / job_status itself. */
enum { MI355_EXP_GFX1151 = 0, MI355_EXP_DECLARED = 1,
       MI355_EXP_LIBM = 2 };   /* router softmax only: the C library's expf as the reference's router test oracle uses it
                                  (tests/hip_moe_route_launcher_tests.hip:329), restated in double precision on the device */

const char* mi355_last_error(void);
const char* mi355_version(void);
/* Numerical identity strings this library implements (the caller opts in by passing them back, as with
 * Request::approved_numerical_identity, include/strix/moe_q4k_a8_contract.hpp:24-26,104-116). */
const char* mi355_numerical_identity(uint32_t weight_type, int down);

/* ------------------------------------------------------------------------------------------------------
 * Block decode. Replaces strix::ggml_dequant::dequantize_row (include/strix/ggml_dequant.hpp:41,
 * src/ggml_dequant.cpp:84-87,119-130). Row r is read at rows + r * row_stride_bytes and written at
 * out + r * out_stride (floats). Bitwise the reference's values.
 */
int32_t mi355_dequantize_rows(uint32_t weight_type, const void* rows, uint64_t row_stride_bytes, uint32_t n_rows,
                              uint32_t elements, float* out, uint64_t out_stride, mi355_stream stream);

/* Writers used to build synthetic weights on the device. Q8_0 = strix::q8_0::quantize_group
 * (include/strix/q8_0_rule.hpp:25-33) with the scale stored as fp16 (round to nearest even). The Q4_K writer has no
 * counterpart in the reference (it only reads GGUF): per 32-value sub-block scale = (max - min) / 15 and offset = -min
 * (min clamped to <= 0), super-block d = max scale / 63 and dmin = max offset / 63 stored as fp16, 6-bit sub-block factors
 * and 4-bit codes by round-to-nearest against the fp16-rounded d / dmin. */
int32_t mi355_quantize_weight_rows(uint32_t weight_type, const float* x, uint32_t n_rows, uint32_t elements,
                                   void* out, mi355_stream stream);

/* ------------------------------------------------------------------------------------------------------
 * RMSNorm of fp32 rows. Replaces strix::cpu::Kernels::rmsnorm_f32 (src/cpu/core/backend.hpp:71-72,
 * src/cpu/core/reference.cpp:86-103): ReductionOrder::lane_strided_fma_lds_halving with 256 lanes for n >= 512 and 128
 * below (backend.hpp:91): lane l runs the fma chain over x[l], x[l + L], ..., the partial sums are halved pairwise
 * (l, l + h), r = 1 / sqrt(sum / n + eps), y = (x * r) * w (w may be NULL: y = x * r). Rows are dense: [rows][n].
 */
int32_t mi355_rmsnorm_f32(const float* x, const float* w, uint32_t n, float eps, float* y, uint32_t rows,
                          mi355_stream stream);

/* ------------------------------------------------------------------------------------------------------
 * A8 activation quantiser. Replaces strix::cpu::Kernels::quantize_a8 (src/cpu/core/backend.hpp:68-69,
 * src/cpu/core/reference.cpp:35-55): groups of 32, delta = amax / 127 (1 for an all-zero group or amax < 2^-119),
 * code = rint(x / delta) clamped to +-127, per-group code sums. width % 32 != 0 -> MI355_E_INVALID_ARGUMENT before any
 * write. x row r at x + r * x_stride_bytes; codes row r at codes + r * width; deltas / sums row r at + r * width / 32.
 * sums and status may be NULL. A non-finite input sets status[r] |= MI355_STATUS_NONFINITE_ACTIVATION.
 */
int32_t mi355_quantize_a8(const void* x, uint32_t input_kind, uint32_t rows, uint32_t width, uint64_t x_stride_bytes,
                          int8_t* codes, float* deltas, int32_t* sums, uint32_t* status, mi355_stream stream);

/* ------------------------------------------------------------------------------------------------------
 * Dense Q8_0 x A8 product. Field for field strix::cpu::Q8a8View (src/cpu/core/backend.hpp:52-59); replaces
 * strix::cpu::Kernels::gemv_q8_0_a8 (src/cpu/core/backend.hpp:70, src/cpu/core/reference.cpp:57-84):
 * group g into lane g % 32 ascending, float(dot) * (scale_w * delta_x), tree32, optional out += product.
 * in % 32 != 0 -> MI355_E_INVALID_ARGUMENT before any write.
 */
typedef struct mi355_q8a8_view {
    const uint8_t* weight;   /* output o at weight + o * row_bytes (2-byte aligned) */
    const int8_t* codes;     /* A8 codes, row r at codes + r * x_stride */
    const float* deltas;     /* deltas[r * (x_stride / 32) + k / 32] */
    float* out;              /* out[r * out_stride + o] */
    uint32_t row_bytes, in, count, rows, x_stride, out_stride;
    uint32_t accumulate;
} mi355_q8a8_view;
int32_t mi355_gemv_q8_0_a8(const mi355_q8a8_view* view, mi355_stream stream);

/* The reference's DENSE A8 profile of its Q8_0 projections (numerical profile dense-a8-q80-v1: the shared expert and the other dense
 * sites of the decode step, src/hip_shared_expert_launcher.hip:1084-1142, row contract src/hip_q8_rows_gemv.hpp:1155-1170, stated on
 * the host in tests/dense_a8_small_reference_tests.cpp:93-104):
 *   quantiser, per block of 32: any non-finite x -> delta = NaN (0x7fc00000), codes 0; amax = max |x|; tiny = 0 < amax < 2^-119;
 *     delta = (amax == 0 || tiny) ? 1 : amax / 127; code = tiny ? 0 : clamp(rint(x / delta), -127, 127)  (no status word, no sums);
 *   product: acc = +0, then acc = fma(float(d_w[n][b]) * delta[r][b], float(sum_k q_w[n][b][k] * code[r][b][k]), acc) over the blocks b
 *     in ascending order; y = isnan(acc) ? 0x7fc00000 : acc.
 * The view is mi355_q8a8_view (accumulate must be 0; in % 64 == 0, in <= 8192, weight rows 4-byte aligned). With the shared gate
 * (mi355_shared_gate), the SiLU of mi355_swiglu_quantize's h_out and one multiply by the gate these are the steps of the reference's
 * shared expert in that profile. */
int32_t mi355_dense_a8_quantize(const void* x, uint32_t input_kind, uint32_t rows, uint32_t width, uint64_t x_stride_bytes, int8_t* codes,
                                float* deltas, mi355_stream stream);
int32_t mi355_gemv_q8_0_a8_chain(const mi355_q8a8_view* view, mi355_stream stream);

/* ------------------------------------------------------------------------------------------------------
 * Router. Replaces the Qwen route launcher (include/strix/hip_moe_route_launcher.hpp:16-30,
 * src/hip_moe_route_launcher.hip:322-365) with the host policy's bits (include/strix/moe/route_policy.hpp:99-156):
 * logits by the per-expert ascending fma chain (or the 32-lane strided sum + butterfly), optional per-expert logit
 * bias, softmax (max, exp(z - max), ascending sum, divide) with Math::exp = the declared exp
 * (include/strix/ds41_moe.hpp:38-54), k selection passes in ascending id (greater score wins, lower id on ties),
 * weights (s / (sum_in_selection_order + renorm_eps)) * scale.
 */
typedef struct mi355_route_policy {
    uint32_t experts, top_k;          /* experts <= 1024, top_k <= 16 */
    uint32_t logits_order;            /* MI355_LOGITS_* */
    float renorm_eps, scale;
    uint32_t renormalize;
    uint32_t renorm_single;           /* the weights are renormalised when renormalize && (top_k > 1 || renorm_single)
                                         (include/strix/moe/route_policy.hpp:146) */
    uint32_t exp_kind;                /* Math::exp of the softmax: MI355_EXP_DECLARED (include/strix/ds41_moe.hpp:38-54),
                                         MI355_EXP_LIBM or MI355_EXP_GFX1151 */
    uint32_t shared_experts;          /* 0..4 always-on experts behind the routed ones: ids / weights rows are then
                                         [top_k + shared_experts] wide, slot top_k + s holds expert id experts + s with weight 1
                                         (the shared expert of a layer stored as one more expert of the same tensors) */
    const float* shared_slot_weights; /* NULL, or device fp32 [rows][shared_experts]: the weight of each always-on slot in the place of 1 -
                                         the shared expert's sigmoid gate (mi355_shared_gate). An always-on slot enters the ordered
                                         combine as acc + (weight * value), product and sum rounded separately: the reference scales
                                         the shared expert's output by its gate (one multiply, src/hip_shared_expert_launcher.hip:727,
                                         :779) and adds that row to the routed sum (include/strix/moe/combine.hpp:56); with weight 1
                                         this is acc + value */
} mi355_route_policy;
/* x: [rows] activations (input_kind), row r at x + r * x_stride_bytes. router_weight: fp32 [experts][hidden].
 * logit_bias: fp32 [experts] or NULL. ids / weights: [rows][top_k + shared_experts]. scores: [rows][experts] workspace AND output. */
int32_t mi355_moe_route(const mi355_route_policy* policy, const void* x, uint32_t input_kind, uint32_t rows,
                        uint32_t hidden, uint64_t x_stride_bytes, const float* router_weight, const float* logit_bias,
                        uint32_t* ids, float* weights, float* scores, mi355_stream stream);

/* The host executor's per-row A8 image and assignment (RowA8, Assignment: src/cpu/core/routed_expert.hpp:41-49), device pointers. */
typedef struct mi355_row_a8 { const int8_t* codes; const float* deltas; const int32_t* sums; } mi355_row_a8;
typedef struct mi355_expert_assignment { uint32_t row, slot, expert; } mi355_expert_assignment;

/* ------------------------------------------------------------------------------------------------------
 * Routed experts. The whole-layer form follows the reference's host API for one MoE layer
 * (include/strix/cuda/qwen_moe.hpp:55-110: Rows / Weights, enqueue_prologue / csr / project / down / merge) and
 * computes what strix::cpu::expert::reference_run computes (src/cpu/core/routed_expert.cpp:264-300) with Q4_K or Q5_K gate/up
 * and Q4_K down (down rows by the gate/up row contract: src/moe_a8_down_contract.cpp:146) or the host executor's own down
 * formats, Q8_0 and Q5_1 blocks of 32 (src/cpu/core/routed_expert.hpp:28, routed_expert.cpp:110-144), or Q6_K down rows
 * (src/moe_a8_down_contract.cpp:18-37, 147-158). The single-row C1 forms of
 * include/strix/hip_moe_q4k_a8_probe.hpp:12 and include/strix/hip_moe_a8_down.hpp:11-30 are rows = 1.
 */
typedef struct mi355_moe_weights {
    uint32_t hidden;      /* multiple of 256 */
    uint32_t ffn;         /* intermediate rows computed by this call (a TP rank: its share), multiple of 256 */
    uint32_t experts, top_k;
    uint32_t gate_type, down_type;                    /* gate/up MI355_TYPE_Q4_K or Q5_K; down Q4_K, Q8_0, Q5_1 or Q6_K
                                                         (mi355_moe_enqueue_prefill_f16: Q4_K, Q5_K or Q8_0 for either) */
    const uint8_t *gate, *up, *down;                  /* GGUF order [experts][ffn][hidden/256], [experts][hidden][ffn/256 or ffn/32 blocks] */
    uint64_t gate_expert_stride, gate_row_stride;     /* bytes; 0 = dense GGUF order. 16-byte multiples (Q6_K down: 2) */
    uint64_t down_expert_stride, down_row_stride;     /* a TP rank reads the first ffn/256 blocks of each down row */
    uint32_t exp_kind;                                /* MI355_EXP_GFX1151 or MI355_EXP_DECLARED, used by SiLU */
    float swiglu_limit;                               /* the SwiGLU clamp trait (include/strix/moe/activation_policy.hpp:22-24,
                                                         DownRequest::swiglu_limit include/strix/moe_a8_down_contract.hpp:45):
                                                         finite L > 0: g = min(g, L), u = clamp(u, -L, L) before silu(g) * u, the
                                                         fail-closed check stays on the raw projections; +infinity (or 0, the
                                                         zero-initialised default) = no clamp; anything else is rejected */
} mi355_moe_weights;

typedef struct mi355_moe_rows {
    const void* input; uint32_t input_kind; uint64_t input_stride;  /* [rows] activations, stride in bytes */
    const uint32_t* routes;          /* [rows][top_k] expert ids */
    const float* route_weights;      /* [rows][top_k] */
    int8_t* codes; float* deltas; int32_t* sums;      /* A8 image of the input: [rows][hidden], [rows][hidden/32] x2 */
    uint32_t* status;                /* [rows] sticky status words (cleared by the prologue) */
    float* gate_out; float* up_out; float* h_out;     /* optional [rows][top_k][ffn] fp32 intermediates, may be NULL */
    int8_t* down_codes; float* down_deltas; int32_t* down_sums;   /* A8 image of h: [rows][top_k][ffn], [..][ffn/32] x2 */
    float* rawdots;                  /* [rows][top_k][hidden] unweighted down outputs */
    const float* base;               /* optional [rows][hidden] added by the merge (shared expert output) */
    float* output; uint64_t output_stride;            /* [rows][hidden] fp32, stride in floats */
    uint32_t* plan;                  /* mi355_moe_plan_words(experts, rows, top_k) words, 16-byte aligned */
    uint32_t* job_status;            /* 1 word of job-wide flags: MI355_STATUS_NONFINITE_PROJECTION when any row's gate, up or h
                                        was non-finite (the down phase is then skipped and no row is published). An invalid
                                        route or a non-finite input flags only its own row (status[row]); the reference's
                                        summary word fails the whole job for those too */
    void* h_f16;                     /* optional workspace of mi355_moe_prefill_f16_workspace_bytes() bytes, 16-byte aligned,
                                        used only by mi355_moe_enqueue_prefill_f16 (h in fp16 and sub-block sums) */
} mi355_moe_rows;

size_t mi355_moe_plan_words(uint32_t experts, uint32_t rows, uint32_t top_k);
size_t mi355_moe_prefill_f16_workspace_bytes(uint32_t hidden, uint32_t ffn, uint32_t rows, uint32_t top_k);

/* prologue: clear status, validate routes and route weights, A8-quantise the input rows. */
int32_t mi355_moe_enqueue_prologue(const mi355_moe_weights*, const mi355_moe_rows*, uint32_t rows, mi355_stream);
/* csr: the expert grouping plan - assignments (row, slot) of each expert, stable rows-then-slots order
 * (src/hip_moe_q4k_a8_probe.hip:91-147). */
int32_t mi355_moe_enqueue_csr(const mi355_moe_weights*, const mi355_moe_rows*, uint32_t rows, mi355_stream);
/* project: gate and up rows of every touched expert, SwiGLU, A8 re-quantisation of h per 32 outputs. */
int32_t mi355_moe_enqueue_project(const mi355_moe_weights*, const mi355_moe_rows*, uint32_t rows, mi355_stream);
/* down: rawdots[row][slot][hidden]; skipped on the device when any row reported a non-finite projection. */
int32_t mi355_moe_enqueue_down(const mi355_moe_weights*, const mi355_moe_rows*, uint32_t rows, mi355_stream);
/* merge: ordered combine of the slots (+ base) into output; form = MI355_COMBINE_*. A flagged row, and every row of a job
 * whose down phase was skipped, is left unwritten. */
int32_t mi355_moe_enqueue_merge(const mi355_moe_weights*, const mi355_moe_rows*, uint32_t rows, uint32_t form,
                                mi355_stream);
/* prologue + csr + project + down + merge. */
int32_t mi355_moe_enqueue(const mi355_moe_weights*, const mi355_moe_rows*, uint32_t rows, uint32_t combine_form,
                          mi355_stream);

/* The combine as an operator of its own (strix::moe_core::enqueue_combine / enqueue_combine_rounded_eo,
 * src/moe_core/route_wave_kernel.hpp:98-160; host restatement strix::moe::combine_ref, include/strix/moe/combine.hpp:36-59).
 * eo [rows][top_k][width], w [rows][top_k], base [rows][width], y [rows][width], all dense fp32 on the device.
 *   MI355_COMBINE_FMA_SLOT_ORDER: acc = fma(w_k, e_k, acc) in slot order, y = acc + base; w and base are required.
 *   MI355_COMBINE_BF16_STEPS:     acc = bf16(acc + term_k), term_k = w ? bf16(e_k * w_k) : e_k (w NULL: unit weights);
 *                                 y = base ? bf16(acc + base) : acc. round_eo != 0 reads every e_k as bf16(e_k), the value a
 *                                 separate rounding launch over eo would have stored (bf16-steps form only).
 * bf16() rounds to nearest even into the upper 16 bits and passes a NaN through unchanged. No status words: like the
 * reference operator this one only computes. rows == 0 is a no-op. */
int32_t mi355_moe_enqueue_combine(uint32_t form, uint32_t rows, uint32_t top_k, uint32_t width, const float* w, const float* eo,
                                  const float* base, float* y, uint32_t round_eo, mi355_stream);

/* The same layer with its router in front (the reference's per-layer walk moe_route -> moe_experts -> moe_combine,
 * include/strix/execution_plan.hpp:22-25): rows->routes and rows->route_weights are OUTPUTS of this call (the selected ids
 * and weights), scores is a [rows][experts] workspace and output. For rows <= 16 the router, the A8 prologue and the expert
 * plan run in ONE launch (the workgroup that completes a row's logits also selects its experts and writes the row's work
 * items: one item per assignment, in assignment order; the CSR fields of the plan are not written), followed by project,
 * down and merge (down and merge share a launch up to a few rounds of that launch's workgroups on the chip). Batches of
 * 8 .. 128 assignments (1 .. 16 rows of top-8) over Q4_K experts of hidden <= 2048 run as two launches: the gate / up sweeps start on experts picked from
 * lane-parallel logits while the reference's logit chains, softmax and selection run beside them in the same launch; an
 * assignment whose early pick differs from the exact one is repaired before the down rows (copied from the slot that held its
 * expert, or swept again on the exact expert), so the results
 * are the exact router's in every case (the unweighted-output view serves as the early logits' scratch until then). Where an
 * expert's gate + up rows exceed 4 MB (and the batch is too large for the 16-rows-per-wavefront sweep) such a batch goes the
 * staged way instead - router, prologue, plan with up to two rows per work item - so that two rows that chose one expert
 * share one sweep of its weights; the results are the same bits. rows->plan must be zero-filled once when it is allocated; every launch leaves its ticket words zero, and
 * they sit at a fixed place, so one workspace serves calls with any row count up to the one it was sized for. */
int32_t mi355_moe_enqueue_layer(const mi355_route_policy* policy, const float* router_weight, const float* logit_bias,
                                float* scores, const mi355_moe_weights*, const mi355_moe_rows*, uint32_t rows,
                                uint32_t combine_form, mi355_stream);
/* mi355_moe_enqueue_layer as its two halves, for a caller that places other work between them (the reference's walk enqueues
 * moe_route / moe_experts and moe_combine as separate steps, include/strix/execution_plan.hpp:22-25) or times them apart:
 * front = router, A8 prologue, expert plan, gate / up + SwiGLU + A8 of h; back = down rows + ordered combine on what the front
 * call left in the row views. Both take the arguments of the whole call; front followed by back on one stream is that call. */
int32_t mi355_moe_enqueue_layer_front(const mi355_route_policy* policy, const float* router_weight, const float* logit_bias,
                                      float* scores, const mi355_moe_weights*, const mi355_moe_rows*, uint32_t rows,
                                      uint32_t combine_form, mi355_stream);
int32_t mi355_moe_enqueue_layer_back(const mi355_route_policy* policy, const float* router_weight, const float* logit_bias,
                                     float* scores, const mi355_moe_weights*, const mi355_moe_rows*, uint32_t rows,
                                     uint32_t combine_form, mi355_stream);

/* Test aid of the decode layer (no counterpart in the reference). A decode batch on the 64-row sweeps picks its experts from
 * lane-parallel logits and runs the reference's logit chain, softmax and selection beside the
 * projection; where the two choices differ the assignment is recomputed on the exact expert before the down rows. The results
 * are the exact router's either way. amount != 0 displaces the early logits (by amount * 1e-3 * a per-expert integer in
 * -8..7) so that a test can make the choices differ; 0 (the default) restores them. Process-wide; not for production use. */
void mi355_debug_early_route_perturb(uint32_t amount);
/* Test and measurement aid (no counterpart in the reference): the down rows + combine launch of a decode batch streams dense rows of at
 * most four super-blocks as contiguous stages; on = 0 sends them through the 144-byte-block stages that every other shape uses, so that
 * the two forms can be compared (same bits). Process-wide; the default is on. */
void mi355_debug_down_merge_flat(uint32_t on);

/* The scalar gate of an always-on shared expert (tensor ffn_gate_inp_shexp, fp32 [hidden]): gate[row * gate_stride] =
 * 1 / (1 + exp(-dot(x[row], scalar_weight))), the reference's shared_gate_dot (src/hip_shared_expert_launcher.hip:624-645): 256
 * thread-strided fma chains (thread t takes features t, t + 256, ... in ascending order), the 256-leaf halving tree
 * s[l] + s[l + h], h = 128 .. 1 (src/core/ordered_reduce.hpp:8-16), the device expf (exp_kind MI355_EXP_GFX1151 is the
 * reference's) and a correctly rounded division. x: rows of input_kind, row r at x + r * x_stride_bytes. gate_stride in floats:
 * [rows][shared_experts] for the policy's shared_slot_weights, or 1 for the route weights of a top-1 shared-expert layer call. */
int32_t mi355_shared_gate(const void* x, uint32_t input_kind, uint32_t rows, uint32_t hidden, uint64_t x_stride_bytes,
                          const float* scalar_weight, uint32_t exp_kind, float* gate, uint64_t gate_stride, mi355_stream);

/* The layer with the RMSNorm of its input inside the first launch (the reference normalises the residual stream in front of
 * the MoE, src/ops/norm/norm.hpp:40-58, and runs the shared expert beside the routed ones, src/hip_shared_expert_launcher.hip):
 * rows->input holds the raw rows; the router, the A8 image and the experts see y = (x * r) * norm_weight,
 * r = 1 / sqrt(mean(x^2) + norm_eps), bit for bit mi355_rmsnorm_f32 (lane-strided fma chains, LDS halving) followed by
 * mi355_moe_enqueue_layer on y; norm_weight may be NULL (unit scale). normed: fp32 [rows][hidden], receives y (the input of
 * anything else that reads the normalised rows). For rows <= 16 every workgroup of the router / prologue launch derives its
 * row's r itself, so no launch is added; larger batches run one norm launch first.
 * A shared expert stored as expert `experts` of the same tensors is the policy's shared_experts = 1: every row then carries
 * one more slot with weight 1, its gate / up / down rows are swept once per four rows, and the ordered combine adds it last. */
int32_t mi355_moe_enqueue_layer_normed(const mi355_route_policy* policy, const float* router_weight, const float* logit_bias,
                                       float* scores, const float* norm_weight, float norm_eps, float* normed, const mi355_moe_weights*,
                                       const mi355_moe_rows*, uint32_t rows, uint32_t combine_form, mi355_stream);

/* mi355_moe_enqueue_layer with every work buffer inside the library. It has no counterpart in the reference: it is for
 * callers that cannot allocate device memory (code under HIP graph capture, tight serving loops, harnesses that forbid
 * allocation). The caller passes only inputs and outputs: the policy, router and expert tensors, the input rows, and the
 * row outputs routes / route_weights [rows][top_k], status [rows], output [rows][output_stride] (base: optional [rows][hidden]).
 * Router scores, the A8 images, the expert plan, the unweighted down outputs and the job status word live in a device array
 * of about 5.1 MB that is part of the library image (each device the library runs on holds its own copy until the process
 * ends). Limits: rows <= 16, top_k <= 8, hidden <= 8192, ffn <= 4096, experts <= 1024; beyond them the call returns
 * MI355_E_INVALID_ARGUMENT. The call allocates nothing and computes the same bits as mi355_moe_enqueue_layer. Every call on
 * a device shares that device's array: two calls that overlap on one device (different streams or threads) race. The counters
 * inside the array are left zero by every call; when a launch of the sequence fails (MI355_E_HIP) the entry point enqueues their
 * reset itself. The first call on a device (or mi355_static_workspace_prepare) must happen outside a stream capture. */
/* (belongs to mi355_moe_enqueue_layer_static; no counterpart in the reference) Looks up the built-in workspace of the current device
 * and enqueues a kernel that zeroes the counters in it which every call expects to find zero. Call it once per device at set-up -
 * the address look-up is a runtime call that does not belong inside a stream capture; mi355_moe_enqueue_layer_static does the
 * look-up itself on its first call on a device otherwise, so that first call must then happen outside capture - and again
 * after any call of the static entry point was interrupted (a device reset handled by the caller). Allocates nothing. */
int32_t mi355_static_workspace_prepare(mi355_stream);
int32_t mi355_moe_enqueue_layer_static(const mi355_route_policy* policy, const float* router_weight, const float* logit_bias,
                                       const mi355_moe_weights*, const void* input, uint32_t input_kind, uint64_t input_stride,
                                       uint32_t rows, uint32_t* routes, float* route_weights, uint32_t* status, const float* base,
                                       float* output, uint64_t output_stride, uint32_t combine_form, mi355_stream);

/* The routed experts of a prefill batch on the matrix cores - the path's FAST arithmetic class (the reference's
 * bit-changing MMA forms: include/strix/cuda/qwen_moe.hpp:100-101 moe_mma, known_rows::enqueue_prefill
 * include/strix/hip_moe_q4k_a8_known_rows.hpp:109-111). The integers sc * q of the Q4_K blocks (exact in fp16) are multiplied
 * with the fp16 rows by fp16 MFMA with fp32 accumulation, the block scale d applied in fp32 per super-block, the dmin * m
 * terms added as a product over sub-block sums; SiLU uses the declared exp; h is kept in fp16 (rows->h_f16). Results follow the exact-weight product (include/strix/ds41_layer.hpp:96-121) to
 * the library's tolerance (2e-3 of the output rms), NOT the integer-dot class's bits: a caller opts in by calling this
 * entry point. Runs: status clear + route validation, expert plan, gate/up + SwiGLU, down, ordered combine.
 * Requires input_kind = MI355_INPUT_F16, rows->h_f16 (see mi355_moe_prefill_f16_workspace_bytes), hidden % 256 == 0,
 * ffn % 256 == 0.
 * gate_type and down_type may each be MI355_TYPE_Q4_K, MI355_TYPE_Q5_K (the nibble plus a fifth bit: sc * q stays an exact
 * fp16 integer) or MI355_TYPE_Q8_0 here (w = d * code, src/ggml_dequant.cpp:84-87: the codes are the exact operands, d is
 * applied in fp32 to every block's product). An always-on shared expert
 * (src/hip_shared_expert_launcher.hip) is a layer with experts = top_k = 1, every route id 0 and every route weight 1; its
 * output is the next call's rows->base. A row whose h leaves the fp16 range is reported as MI355_STATUS_NONFINITE_PROJECTION. */
int32_t mi355_moe_enqueue_prefill_f16(const mi355_moe_weights*, const mi355_moe_rows*, uint32_t rows, uint32_t combine_form,
                                      mi355_stream);

/* SwiGLU + A8 re-quantisation of h for a dense gate/up pair (the shared expert and the dense FFN):
 * gate / up: fp32 [rows][ffn]; writes h codes / deltas / sums as above and optionally h values.
 * Replaces enqueue_down_activation_quantize (include/strix/hip_moe_a8_down.hpp:18) for rows of gate|up.
 * swiglu_limit: as mi355_moe_weights::swiglu_limit. */
int32_t mi355_swiglu_quantize(const float* gate, const float* up, uint32_t rows, uint32_t ffn, uint32_t exp_kind,
                              float swiglu_limit, int8_t* codes, float* deltas, int32_t* sums, float* h_out, uint32_t* status,
                              mi355_stream stream);

/* ------------------------------------------------------------------------------------------------------
 * The reference's A8 request / bindings boundary (the HIP entry points this library replaces). Field for field:
 *   mi355_device_bytes      = DeviceBytes                  include/strix/moe_q4k_a8_contract.hpp:117
 *   mi355_a8_shape          = Shape                        include/strix/moe_q4k_a8_contract.hpp:104
 *   mi355_a8_request        = Request                      include/strix/moe_q4k_a8_contract.hpp:105-116
 *   mi355_a8_bindings       = Bindings                     include/strix/moe_q4k_a8_contract.hpp:118-120
 *   mi355_a8_down_shape / _request / _bindings = DownShape / DownRequest / DownBindings   include/strix/moe_a8_down_contract.hpp:39-52
 *   mi355_slot_merge_tail   = SlotMergeTail                include/strix/hip_moe_a8_down.hpp:21-29
 * (std::string_view becomes a NUL-terminated string, bool a uint32_t, InputKind one of MI355_INPUT_*.)
 * mi355_a8_validate / mi355_a8_validate_down are the reference's validate / validate_down (src/moe_q4k_a8_contract.cpp:343-372,
 * src/moe_a8_down_contract.cpp:53-82): pure host admission - enabled, the exact numerical identity string of this library
 * (mi355_numerical_identity), bounded dimensions, every view non-null, aligned (16 bytes; down routes / status words: 4) and of EXACTLY the required byte size, every mutable view disjoint from every other view (down:
 * all views pairwise disjoint). Bounds are this library's, wider than the reference's: hidden % 256 <= 16384, rows % 32 <=
 * 16384 (down: intermediate % 128, K-quant % 256), experts <= 1024, top_k <= 16, and logical_rows 1..16: the per-row views
 * (input, routes, codes, deltas, sums, output; down: intermediates, routes, codes, deltas, sums, rawdots) then hold that many
 * contiguous single-row extents, status stays one shared word. Every enqueue validates the whole bundle before its first
 * launch and, as in the reference, never allocates, synchronises, resets or reads back; status words are sticky (OR only).
 */
typedef struct mi355_device_bytes { uintptr_t address; uint64_t bytes; } mi355_device_bytes;
typedef struct mi355_a8_shape { uint32_t hidden, rows, experts, top_k, logical_rows; } mi355_a8_shape;      /* rows = expert intermediate size */
typedef struct mi355_a8_request {
    uint32_t enabled;
    const char* approved_numerical_identity;      /* must equal mi355_numerical_identity(gate_type, 0) */
    uint32_t input;                               /* MI355_INPUT_BF16, MI355_INPUT_F32 (the reference's kinds) or MI355_INPUT_F16 */
    mi355_a8_shape shape;
    uint32_t gate_type, up_type;                  /* 12 or 13, equal */
    uint32_t fused_gate_up;                       /* must be 0 */
    float swiglu_limit;                           /* must be +infinity here: the clamp belongs to the down producer */
} mi355_a8_request;
typedef struct mi355_a8_bindings { mi355_device_bytes input, gate, up, routes, codes, deltas, sums, status, output; } mi355_a8_bindings;
int32_t mi355_a8_validate(const mi355_a8_request*, const mi355_a8_bindings*);
/* enqueue_probe (include/strix/hip_moe_q4k_a8_probe.hpp:12): route check, A8 image of the input row(s), gate and up rows of
 * the chosen experts: output[((row * top_k + slot) * 2 + which) * shape.rows + i] fp32 (which 0 = gate, 1 = up), bitwise
 * the reference row contract (src/moe_q4k_a8_contract.cpp:126-140). On a flagged step (status != 0 after the prologue) the
 * projection stores nothing: `output` keeps its previous contents, as in the reference (src/hip_moe_q4k_a8_probe.hip:224-225).
 * With one logical row the image is stored only when the whole row is clean (src/hip_moe_q4k_a8_probe.hip:47-90); with several
 * rows (this library's extension) the image views are unspecified after a flagged step. */
int32_t mi355_a8_enqueue_probe(const mi355_a8_request*, const mi355_a8_bindings*, mi355_stream);
/* enqueue_serial_prologue_probe (include/strix/hip_moe_q4k_a8_probe.hpp:20-23; src/hip_moe_q4k_a8_probe.hip:187-199,503-519): the
 * serial row's step with its glue folded in - one workgroup zeroes clear[0 .. clear_words), checks the routes AND the route
 * weights (an index out of range or a non-finite weight: bit 1, and the quantiser is skipped), quantises, stores the image only
 * when the row is clean, and OVERWRITES the status word with route bits | quantiser bits; then the projection as above.
 * shape.logical_rows must be 1. clear and route_weights ([top_k]) are device pointers, 4-byte aligned. */
int32_t mi355_a8_enqueue_serial_prologue_probe(const mi355_a8_request*, const mi355_a8_bindings*, float* clear, uint32_t clear_words,
                                               const float* route_weights, mi355_stream);
/* enqueue_quantize_only (include/strix/hip_moe_q4k_a8_probe.hpp:24; src/hip_moe_q4k_a8_probe.hip:540-554): route check and
 * quantiser without the projection. The status word is ORed into; a step whose status is already set (or whose route check sets it)
 * is not quantised and stores nothing. shape.logical_rows must be 1; every binding is validated as for the probe. */
int32_t mi355_a8_enqueue_quantize_only(const mi355_a8_request*, const mi355_a8_bindings*, mi355_stream);

typedef struct mi355_a8_down_shape { uint32_t hidden, intermediate, experts, top_k; } mi355_a8_down_shape;
typedef struct mi355_a8_down_request {
    uint32_t enabled;
    const char* approved_numerical_identity;      /* must equal mi355_numerical_identity(weight_type, 1) */
    mi355_a8_down_shape shape;
    uint32_t weight_type;                         /* 7 (Q5_1), 8 (Q8_0), 12 (Q4_K) or 14 (Q6_K) */
    float swiglu_limit;                           /* +infinity (none) or finite > 0: the clamped producer */
} mi355_a8_down_request;
/* intermediates: per (row, slot) [gate I | up I] fp32 (the probe's output); the producer replaces ONLY gate with h. */
typedef struct mi355_a8_down_bindings {
    mi355_device_bytes intermediates, weights, routes, codes, deltas, sums, rawdots, status, aggregate_status;   /* aggregate_status may be {0, 0} */
} mi355_a8_down_bindings;
int32_t mi355_a8_validate_down(const mi355_a8_down_request*, const mi355_a8_down_bindings*, uint32_t logical_rows);
/* enqueue_down_activation_quantize (include/strix/hip_moe_a8_down.hpp:18): h = silu(g) * u (clamp trait applied first) and its
 * A8 image; invalid route -> status |= 1, non-finite g / u / h -> status |= 8, either -> aggregate_status |= 16.
 * exp_kind: MI355_EXP_* of the SiLU (the reference's device expf is MI355_EXP_GFX1151). */
int32_t mi355_a8_enqueue_down_activation_quantize(const mi355_a8_down_request*, const mi355_a8_down_bindings*, uint32_t logical_rows,
                                                  uint32_t exp_kind, mi355_stream);
/* enqueue_down_rawdots (include/strix/hip_moe_a8_down.hpp:19): rawdots[(row * top_k + slot) * hidden + o], unweighted. */
int32_t mi355_a8_enqueue_down_rawdots(const mi355_a8_down_request*, const mi355_a8_down_bindings*, uint32_t logical_rows, mi355_stream);
/* The same for one row, then the ordered expert-slot merge, the finite / commit test and the first-error record
 * (include/strix/moe_slot_merge.hpp:1-12,47-55; src/hip_moe_q4k_a8_probe.hip:825-897): accumulation[o] = fma chain over the slots
 * from +0 in slot order; any |value| with bits >= 0x7f800000 (bf16_commit: >= 0x7f7f8000, i.e. also what rounds to bf16
 * infinity) fails the step: status |= 8 and nothing is committed; a clean step stores output (fp32, or bf16 round to nearest
 * even when output_bf16); record = DeferredMoeFirstError {domain, bits} keeps the first non-zero status. tickets is accepted
 * for signature parity and left untouched (the merge is a launch of its own here). */
typedef struct mi355_slot_merge_tail {
    uint32_t* tickets; const float* route_weights; float* accumulation; void* output;
    uint32_t output_bf16, bf16_commit; void* record; uint32_t domain;
} mi355_slot_merge_tail;
int32_t mi355_a8_enqueue_down_rawdots_merge(const mi355_a8_down_request*, const mi355_a8_down_bindings*, const mi355_slot_merge_tail*, mi355_stream);

/* Union rows form: a verify window of R <= 8 rows, each with its top_k <= 16 routes, reads every distinct expert ONCE
 * (include/strix/moe/expert_union.hpp:1-57). `plan` is the expert-union plan, MI355_UNION_PLAN_BYTES in the caller's memory:
 * header {count, rows, top_k, 0} (4 x uint32), then 128 entries {uint32 expert, uint8 slot[8]}: the distinct experts in
 * first-occurrence order of (row, slot) ascending and, per row, the slot that row holds the expert in (0xff: not chosen).
 * mi355_a8_enqueue_probe_union builds it on the device (byte for byte expert_union::build for the `count` entries; the
 * others hold expert 0 and 0xff slots), the down entry points read it. Per (row, slot, output) the arithmetic is the
 * single-row form's: every output is bitwise that of R single-row calls.
 *   mi355_a8_validate_union / _down_union = validate_union / validate_down_union   src/moe_q4k_a8_contract.cpp:373-405,
 *                                                                                  src/moe_a8_down_contract.cpp:83-113
 *   mi355_a8_enqueue_probe_union / _down_activation_quantize_union / _down_rawdots_union
 *                                         = the entry points of the same names     src/hip_moe_q4k_a8_probe.hip:1172-1221
 * Admission as in the reference: R <= 8, K <= 16, Q4_K gate / up (down: Q4_K or Q6_K), every row slice of the per-row views
 * a single-row bundle of its own (16-byte aligned: top_k % 4 == 0 when R > 1), the plan view 16-byte aligned, exactly
 * MI355_UNION_PLAN_BYTES and disjoint from every other view. (The reference's hidden <= 1536 bound is its kernel's register
 * staging; hidden is bounded here as in mi355_a8_validate.) An expert id >= experts, or one named twice by the same row,
 * sets MI355_STATUS_INVALID_ROUTE in the status word, leaves count = 0 and nothing is projected. */
#define MI355_UNION_MAX_ROWS 8u
#define MI355_UNION_MAX_TOP_K 16u
#define MI355_UNION_PLAN_BYTES 1552u
int32_t mi355_a8_validate_union(const mi355_a8_request*, const mi355_a8_bindings*, mi355_device_bytes plan);
int32_t mi355_a8_enqueue_probe_union(const mi355_a8_request*, const mi355_a8_bindings*, mi355_device_bytes plan, mi355_stream);
int32_t mi355_a8_validate_down_union(const mi355_a8_down_request*, const mi355_a8_down_bindings*, uint32_t rows, mi355_device_bytes plan);
int32_t mi355_a8_enqueue_down_activation_quantize_union(const mi355_a8_down_request*, const mi355_a8_down_bindings*, uint32_t rows,
                                                        mi355_device_bytes plan, uint32_t exp_kind, mi355_stream);
int32_t mi355_a8_enqueue_down_rawdots_union(const mi355_a8_down_request*, const mi355_a8_down_bindings*, uint32_t rows, mi355_device_bytes plan,
                                            mi355_stream);

/* ------------------------------------------------------------------------------------------------------
 * The strided form of the per-row views: the reference's multi-row entry binds every view as Strided<T>{base, stride in
 * bytes}, row r at base + r * stride (Rows, include/strix/cuda/qwen_moe.hpp:34-37,55-76 = the views of the HIP
 * KnownMoePrefillPrepared, src/hip_moe_experts_launcher.hip:2884-2904); a caller that holds such buffers binds them here
 * without a copy. Field for field Rows, with this library's plan words in the place of the reference's Csr views and the
 * job word (the reference's csr.summary[0]) named. Per row: input [hidden] (input_kind; the reference: bf16), routes
 * [top_k], route_weights [top_k], codes [hidden], deltas / sums [hidden / 32], status [1], intermediates [top_k][2][ffn]
 * (h in the place of gate | up; base may be null), accumulation [>= hidden floats], down_codes [top_k][ffn], down_deltas /
 * down_sums [top_k][ffn / 32], rawdots [top_k][hidden], output [hidden] (output_kind: MI355_INPUT_BF16 as in the reference,
 * or MI355_INPUT_F32). Every base and stride is a multiple of 16 bytes (routes, route_weights, status: 4).
 * Stages, same names and order as the reference (include/strix/cuda/qwen_moe.hpp:96-110):
 *   prologue  zero accumulation[0 .. clear_words), check the routes (bad id or non-finite weight: status = 1, row not
 *             quantised), A8 image of the input with the probe contract's quantiser (no tiny-group rule; non-finite value:
 *             bit 2; delta underflow: bit 4), image stored for a clean row only, status OVERWRITTEN
 *   csr       the expert plan; job_status = OR of every row's status
 *   project / down   the integer-class expert kernels (bitwise mi355_moe_enqueue_project / _down)
 *   merge     nothing for a failed job or row; accumulation[o] = fma chain over the slots in slot order from +0; a value whose
 *             magnitude bits reach 0x7f7f8000 (bf16 output; fp32 output: 0x7f800000) sets bit 8 in the row and the job
 *   commit    record = DeferredMoeFirstError {domain, bits} of the first failed row (a record already set stays,
 *             include/strix/deferred_moe_status.hpp:19-26); a failed job commits nothing; else output = accumulation
 *             (bf16: round to nearest even)
 */
typedef struct mi355_strided { void* base; uint64_t stride; } mi355_strided;
typedef struct mi355_moe_rows_strided {
    mi355_strided input, routes, route_weights, codes, deltas, sums, status, intermediates, accumulation,
                  down_codes, down_deltas, down_sums, rawdots, output;
    uint32_t* plan;              /* mi355_moe_plan_words(experts, rows, top_k) words, 16-byte aligned */
    uint32_t* job_status;        /* one word */
    uint32_t input_kind, output_kind;
} mi355_moe_rows_strided;
int32_t mi355_moe_strided_enqueue_prologue(const mi355_moe_weights*, const mi355_moe_rows_strided*, uint32_t rows, uint32_t clear_words, mi355_stream);
int32_t mi355_moe_strided_enqueue_csr(const mi355_moe_weights*, const mi355_moe_rows_strided*, uint32_t rows, mi355_stream);
int32_t mi355_moe_strided_enqueue_project(const mi355_moe_weights*, const mi355_moe_rows_strided*, uint32_t rows, mi355_stream);
int32_t mi355_moe_strided_enqueue_down(const mi355_moe_weights*, const mi355_moe_rows_strided*, uint32_t rows, mi355_stream);
int32_t mi355_moe_strided_enqueue_merge(const mi355_moe_weights*, const mi355_moe_rows_strided*, uint32_t rows, mi355_stream);
int32_t mi355_moe_strided_enqueue_commit(const mi355_moe_weights*, const mi355_moe_rows_strided*, uint32_t rows, uint32_t* record, uint32_t domain,
                                         mi355_stream);
/* prologue + csr + project + down + merge + commit (enqueue, include/strix/cuda/qwen_moe.hpp:107) */
int32_t mi355_moe_strided_enqueue(const mi355_moe_weights*, const mi355_moe_rows_strided*, uint32_t rows, uint32_t clear_words, uint32_t* record,
                                  uint32_t domain, mi355_stream);

/* Known-prompt prefill over strided rows, FAST class (known_rows::PrefillRows / enqueue_prefill with the separate FP16 prefill
 * contract, include/strix/hip_moe_q4k_a8_known_rows.hpp:75-111): every per-row view is row 0 plus r times its own byte stride.
 * Runs the prologue (zeroes clear[row][0 .. clear_words), checks routes and route weights, OVERWRITES status[row], clears the
 * job word), the expert plan over the rows * top_k assignments (stable: rows then slots), gate / up + SwiGLU and the down rows;
 * rawdots[row][slot][hidden] receives the unweighted outputs and THE CALLER MERGES AND COMMITS (mi355_moe_strided_enqueue_merge /
 * _commit take the same views). rawdots_bf16: every unweighted output is stored once rounded to bfloat16 (as an fp32 value), the
 * stored output of a bfloat16 Linear - the same bits as the fp32 store followed by a rounding pass over rawdots. A non-finite
 * gate / up / h value of a (row, slot) sets bit 8 in the row's status and in the job word; the down rows are then skipped.
 * The views of the integer forms (codes, deltas, sums, down_*) are not part of this bundle: the fp16 form has no A8 image;
 * the integer-class stages over strided rows are mi355_moe_strided_enqueue*. input: fp16 rows; plan: mi355_moe_plan_words words;
 * h_f16: mi355_moe_prefill_f16_workspace_bytes bytes. Arithmetic and tolerance: mi355_moe_enqueue_prefill_f16. */
typedef struct mi355_prefill_rows {
    mi355_strided input, routes, route_weights, status, clear, rawdots;
    uint32_t* plan;
    uint32_t* job_status;
    void* h_f16;
    uint32_t rawdots_bf16;
} mi355_prefill_rows;
int32_t mi355_moe_enqueue_prefill_rows_f16(const mi355_moe_weights*, const mi355_prefill_rows*, uint32_t rows, uint32_t clear_words, mi355_stream);

/* ------------------------------------------------------------------------------------------------------
 * The job form of the host executor (strix::cpu::expert::Job / LayerWeights / Executor, src/cpu/core/routed_expert.hpp:28-61,
 * 79-95): a list of (row, slot, expert) assignments over per-row A8 images, every pointer device memory.
 * rawdots[row * rawdot_row_stride + slot * hidden + o] receives the unweighted down rows; a non-finite gate / up / h value
 * ORs 1 (kNonfinite) into status[row] and the job then computes no down row at all (src/cpu/core/routed_expert.cpp:403-447,
 * 461). The executor object owns the A8 image of h for up to max_assignments assignments of up to max_ffn values
 * (allocated at create, as the host Executor owns its scratch); run allocates nothing and does not synchronise. Expert ids
 * are trusted, as on the host. One job at a time per executor.
 */
typedef struct mi355_layer_weights {
    const uint8_t* gate; const uint8_t* up; const uint8_t* down;      /* GGUF order: gate / up [experts][ffn][hidden / 256], down [experts][hidden][ffn / 32] */
    uint32_t gate_format;        /* GateFormat: 0 = Q4_K, 1 = Q5_K */
    uint32_t down_format;        /* DownFormat: 0 = Q5_1, 1 = Q8_0 */
    uint32_t hidden, ffn;        /* Shape: hidden % 256, ffn % 128 */
} mi355_layer_weights;
typedef struct mi355_expert_job {
    mi355_layer_weights weights;
    const mi355_row_a8* rows;                    /* indexed by assignment.row */
    const mi355_expert_assignment* assignments;
    uint32_t count;
    float* rawdots;
    uint64_t rawdot_row_stride;                  /* in floats */
    uint32_t* status;                            /* per row, OR-ed */
} mi355_expert_job;
void* mi355_executor_create(uint32_t max_assignments, uint32_t max_ffn, uint32_t exp_kind);      /* NULL on failure (mi355_last_error) */
int32_t mi355_executor_run(void* executor, const mi355_expert_job* job, mi355_stream);
void mi355_executor_destroy(void* executor);

/* ------------------------------------------------------------------------------------------------------
 * GGUF v3 container reader and the tensor map of one MoE layer: the data format in front of the path (the reference:
 * strix::gguf::read_file / FileInfo / TensorInfo, include/strix/gguf_reader.hpp:75-117, src/gguf_reader.cpp; the expert
 * tensors as src/qwen_moe_prepared.cpp:104-119 names them). Host code only. open() parses and validates the whole index
 * (version 3, bounded counts, lower-case dotted keys, no duplicate key or tensor name, rank 1..4 with non-zero extents, known
 * tensor types with a pinned storage geometry, general.alignment a non-zero multiple of 8, zero padding, aligned offsets,
 * every tensor inside the file, no overlap) and returns NULL with mi355_last_error() set on any violation. offset is the
 * ABSOLUTE file offset of the tensor's first byte; dims are fastest first, as stored.
 */
typedef struct mi355_gguf_tensor { const char* name; uint32_t n_dims; uint64_t dims[4]; uint32_t ggml_type; uint64_t offset, bytes; } mi355_gguf_tensor;
void* mi355_gguf_open(const char* path);
void mi355_gguf_close(void* file);
uint64_t mi355_gguf_tensor_count(const void* file);
uint64_t mi355_gguf_metadata_count(const void* file);
uint64_t mi355_gguf_alignment(const void* file);
uint64_t mi355_gguf_data_offset(const void* file);
int32_t mi355_gguf_tensor_at(const void* file, uint64_t index, mi355_gguf_tensor* out);
int32_t mi355_gguf_find_tensor(const void* file, const char* name, mi355_gguf_tensor* out);
/* kind: 0 unsigned or boolean (*u), 1 signed (*i), 2 floating (*f), 3 string (*text, valid until close), 4 array (*u = length) */
int32_t mi355_gguf_metadata(const void* file, const char* key, uint32_t* kind, uint64_t* u, int64_t* i, double* f, const char** text);
/* blk.<layer>.ffn_gate_exps / ffn_up_exps [hidden][ffn][experts], ffn_down_exps [ffn][hidden][experts], ffn_gate_inp F32
 * [hidden][experts]; optional (bytes == 0 when absent): ffn_norm F32 [hidden], exp_probs_b F32 [experts], the shared expert
 * ffn_gate_shexp / ffn_up_shexp [hidden][shared_ffn], ffn_down_shexp [shared_ffn][hidden], ffn_gate_inp_shexp F32 [hidden].
 * The expert tensors' bytes are [experts][rows][blocks], exactly what mi355_moe_weights takes. */
typedef struct mi355_gguf_moe_layer_map {
    mi355_gguf_tensor gate, up, down, router, norm, router_bias, shared_gate, shared_up, shared_down, shared_router;
    uint32_t hidden, ffn, experts, shared_ffn, gate_type, down_type;
} mi355_gguf_moe_layer_map;
int32_t mi355_gguf_moe_layer(const void* file, uint32_t layer, mi355_gguf_moe_layer_map* out);

#ifdef __cplusplus
}
#endif
#endif
