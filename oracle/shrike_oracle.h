/*
 * TEST INFRASTRUCTURE — NOT PRODUCT CODE.
 *
 * Scalar CPU restatement of the arithmetic of Shrike's routed-expert path
 * (router -> top-k -> slot resolve -> group-affine int4/int8 SwiGLU FFN ->
 * weighted combine + shared expert, and the prefill reduce). Only tests/,
 * __graft_entry__.smoke() and bench.py's cpu_baseline leg may load it, and only
 * as the checker. Each function cites the reference file:line it follows
 * (paths relative to the reference checkout).
 *
 * Pinned by tests/test_oracle_cpu.py: bit-equality with the reference's own C
 * kernel compiled in place (oracle/_ref), the reference tests' known answers,
 * closed forms and fp64 brute force from the format's definition.
 *
 * PARITY UNPINNED: the rounding points and the summation order of the Metal
 * kernels (simd_sum order, half-precision x-sums, fast::exp, and exactly where
 * orc_shared_*, orc_moe_phase2 and orc_router_logits round or add) cannot be
 * pinned bit for bit without running Metal. These functions put the fp16
 * roundings where the Metal sources put them and accumulate in fp32; outputs
 * that depend on them are compared within tolerance, never bit for bit. The
 * bit pattern of the fp32 router logits is this build's own definition.
 */
#ifndef SHRIKE_ORACLE_H
#define SHRIKE_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORC_META_BF16 = 0, ORC_META_F16 = 1 };
enum { ORC_ACT_GELU_TANH = 0, ORC_ACT_SILU = 1, ORC_ACT_CLAMPED_SWIGLU = 2 };
enum { ORC_ROUTER_F16 = 0, ORC_ROUTER_AFFINE8 = 8, ORC_ROUTER_AFFINE4 = 4 };

/* sources/Shrike/Kernels/MoE/MoE.swift:4-39, sources/Shrike/Metal/MoE/moe.metal:240-255 */
typedef struct {
    uint32_t gate_w, gate_s, gate_b;
    uint32_t up_w, up_s, up_b;
    uint32_t down_w, down_s, down_b;
    uint32_t gate_ab, up_ab, down_ab;
} orc_offsets;

/* ---- scalar conversions (sources/Shrike/Infrastructure/ModelIO/Quantization.swift:16-28) */
uint16_t orc_f32_to_bf16(float x);
float orc_bf16_to_f32(uint16_t bits);
uint16_t orc_f32_to_f16(float x);
float orc_f16_to_f32(uint16_t bits);

/* ---- blob layout (sources/Shrike/Kernels/CPU/CPUExpertFFN.swift:34-61, generalised to 8-bit) */
void orc_expert_offsets(uint32_t d, uint32_t f, uint32_t bits, int additive_biases,
                        orc_offsets *out, uint64_t *stride_bytes);

/* ---- GEMV bodies */
/* sources/ShrikeKernelsC/int4_affine_gemv.c:114-134 (portable branch), same
 * operation order; meta selects the scale/bias encoding. */
void orc_int4_affine_gemv(const uint8_t *weights, const uint16_t *scales,
                          const uint16_t *biases, int meta, const float *x,
                          size_t rows, size_t n, float *out);
/* generic bits in {4,8}: sources/Shrike/Metal/MoE/moe.metal:46-54,650-672 arithmetic,
 * evaluated in the sequential per-group order of int4_affine_gemv.c:114-134. */
void orc_affine_gemv(const uint8_t *weights, const uint16_t *scales,
                     const uint16_t *biases, int meta, int bits, const float *x,
                     size_t rows, size_t n, float *out);
/* fp64 accumulation of the same product, for error attribution only. */
void orc_affine_gemv_f64(const uint8_t *weights, const uint16_t *scales,
                         const uint16_t *biases, int meta, int bits, const float *x,
                         size_t rows, size_t n, double *out);

/* ---- CPU expert: sources/Shrike/Kernels/CPU/CPUExpertFFN.swift:102-140 */
void orc_cpu_expert_ffn_accumulate(const uint8_t *expert, const orc_offsets *off,
                                   int meta, int bits, const float *x, uint32_t d,
                                   uint32_t f, float route_weight, float *scratch,
                                   float *out);

/* ---- activations: moe.metal:98-105, :233-238, :280-288 */
float orc_glu(float gate, float up, int act);

/* ---- routed decode, GPU semantics.
 * phase 1: moe.metal:779-830 / :950-999 (act rounded to fp16, :829), with the
 * x-sums taken in fp32 (the CPU path's choice, int4_affine_gemv.c:41-53).
 * expert_base[k] == NULL marks a skipped (sentinel) position. */
void orc_moe_phase1(const uint8_t *const *expert_base, const orc_offsets *off,
                    int meta, int bits, int act, int additive_biases,
                    const uint16_t *x_f16, uint32_t d, uint32_t f, uint32_t top_k,
                    uint16_t *acts_f16);
/* phase 2: moe.metal:889-941 / :1008-1057. y = half(residual + sum_k half_w[k]*down_k),
 * hidden = half(hidden + y). */
void orc_moe_phase2(const uint8_t *const *expert_base, const orc_offsets *off,
                    int meta, int bits, int additive_biases,
                    const uint16_t *acts_f16, const uint16_t *routing_w_f16,
                    const uint16_t *residual_f16, uint32_t d, uint32_t f,
                    uint32_t top_k, uint16_t *y_f16, uint16_t *hidden_f16);

/* ---- shared expert (separate resident tensors):
 * int4: sources/Shrike/Metal/Quant/dequant_int4.metal:101-180 (GEMV, fp16 out),
 *       :247-331 (act = half(silu(g)*u) from the fp16 gate/up, down GEMV -> fp16,
 *       optional y*sigmoid(scalar_gate) -> fp16);
 * int8: sources/Shrike/Metal/Quant/dequant_int8.metal:66-107, :109-164.
 * Both families round gate and up through fp16 before the activation. */
typedef struct {
    const uint8_t *w; const uint16_t *s; const uint16_t *b;
} orc_proj;
void orc_shared_gate_up(const orc_proj *gate, const orc_proj *up, int meta, int bits,
                        const uint16_t *x_f16, uint32_t d, uint32_t f, uint16_t *gate_f16,
                        uint16_t *up_f16);
void orc_shared_down(const orc_proj *down, int meta, int bits, int act, const uint16_t *gate_f16,
                     const uint16_t *up_f16, uint32_t d, uint32_t f,
                     const uint16_t *scalar_gate_f16, uint16_t *h1_f16);
void orc_shared_expert(const orc_proj *gate, const orc_proj *up, const orc_proj *down,
                       int meta, int bits, int act, const uint16_t *x_f16, uint32_t d,
                       uint32_t f, const uint16_t *scalar_gate_f16 /* NULL = ungated */,
                       uint16_t *h1_f16);

/* The per-row scalar gate of the shared expert for a block of tokens,
 * sources/Shrike/Metal/MoE/moe.metal:1154-1207: one 8-bit weight row against `rows`
 * activation rows (eight partial sums added in order, fp16 out), and y[row,:] *= sigmoid(gate[row]). */
void orc_shared_scalar_gate_rows(const uint8_t *w, const uint16_t *scales, const uint16_t *biases, int meta,
                                 const uint16_t *x_f16, uint32_t x_stride, uint32_t rows, uint32_t d,
                                 uint16_t *gate_f16);
void orc_sigmoid_scalar_mul_rows(uint16_t *y_f16, const uint16_t *gate_f16, uint32_t d, uint32_t rows);

/* ---- router.
 * Logits: moe.metal:324-364 arithmetic (x = half(hidden) * bf16(effective_scale)).
 * The reference leaves the cross-lane summation order open (simd_sum, :362); this
 * restatement fixes it: 64 partial sums, partial l taking the 16-byte weight chunks
 * c = l, l+64, ... in order with one fused multiply-add per element (affine:
 * per chunk dot and x-sum, then fma(scale, dot, acc), fma(bias, xsum, acc)), the
 * partials combined by the butterfly v[l] += v[l^o], o = 32,16,8,4,2,1. */
void orc_router_logits(const void *weights, const uint16_t *scales, const uint16_t *biases,
                       int router_kind, int meta, const uint16_t *hidden_f16,
                       const uint16_t *effective_scale_bf16, uint32_t num_experts,
                       uint32_t d, float *logits);
/* moe.metal:419-491: insertion top-K, ties to the lower index; softmax over the
 * selected or (sigmoid) renormalised original sigmoids * scaling; * per-expert scale. */
void orc_router_select(const float *logits, const uint16_t *per_expert_scale_bf16,
                       const uint16_t *bias_bf16, uint32_t num_experts, uint32_t top_k,
                       int sigmoid_scores, float scaling, uint32_t *out_indices,
                       uint16_t *out_weights_f16);
/* moe.metal:121-151 */
uint32_t orc_classify(const uint32_t *topk, const uint64_t *residency, uint32_t top_k,
                      uint32_t num_experts, uint32_t *hit_count, uint32_t *hit_positions,
                      uint32_t *miss_count, uint32_t *miss_positions, uint32_t *miss_experts,
                      uint32_t *resolved_slots);

/* ---- prefill reduce: sources/Shrike/Metal/Prefill/prefill.metal:624-645 */
void orc_prefill_reduce(const uint16_t *partials_f16, const uint16_t *weights_f16,
                        uint32_t t, uint32_t top_k, uint32_t d, uint16_t *h2_f16);
/* residual_add_fp16: sources/Shrike/Metal/Primitives/utility.metal:94-103 */
void orc_residual_add_f16(uint16_t *hidden, const uint16_t *delta, size_t n);
void orc_residual_add_rmsnorm_bf16w(uint16_t *hidden, const uint16_t *delta, const uint16_t *weight_bf16,
                                    uint16_t *out, uint32_t d, float eps);

/* ---- whole-layer timing helper for the CPU baseline (one task per expert,
 * sources/Shrike/Kernels/CPU/CPUExpertFFN.swift:10-14 describes 6 threads). */
void orc_cpu_layer_fp32(const uint8_t *const *experts, const float *route_weights,
                        uint32_t n_experts, const orc_offsets *off, int meta, int bits,
                        const float *x, uint32_t d, uint32_t f, uint32_t threads, float *out);

#ifdef __cplusplus
}
#endif
#endif
