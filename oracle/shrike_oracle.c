/*
 * TEST INFRASTRUCTURE — NOT PRODUCT CODE. See shrike_oracle.h.
 *
 * Build with -ffp-contract=off: several functions below are compared bit for
 * bit with the reference's C file compiled the same way, so no product may be
 * fused into a following add unless fmaf() is written out.
 */
#include "shrike_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#define ORC_GROUP 64u

/* ------------------------------------------------------------------ scalars */

/* Quantization.swift:17-24: round-half-to-even on the upper 16 bits, no NaN case. */
uint16_t orc_f32_to_bf16(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7FFFu + lsb;
    return (uint16_t)(u >> 16);
}

float orc_bf16_to_f32(uint16_t bits) {
    uint32_t u = (uint32_t)bits << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t u;
    if (exp == 0) {
        if (man == 0) {
            u = sign;
        } else { /* subnormal: normalise */
            int shift = 0;
            while ((man & 0x400u) == 0) { man <<= 1; ++shift; }
            man &= 0x3FFu;
            u = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        u = sign | 0x7F800000u | (man << 13);
    } else {
        u = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* IEEE round-to-nearest-even binary32 -> binary16 (what `half(x)` does in MSL). */
uint16_t orc_f32_to_f16(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t absu = u & 0x7FFFFFFFu;
    if (absu >= 0x7F800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | (absu > 0x7F800000u ? 0x200u | ((absu >> 13) & 0x3FFu) : 0u));
    }
    if (absu >= 0x477FF000u) { /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7C00u);
    }
    if (absu < 0x38800000u) { /* below the smallest normal half: subnormal or zero */
        if (absu < 0x33000000u) return (uint16_t)sign; /* < 2^-25 -> 0 (2^-25 itself ties to even 0) */
        int e = (int)(absu >> 23);
        uint32_t man = (absu & 0x7FFFFFu) | 0x800000u;
        int shift = 126 - e; /* man is 24 bits; result = man >> (shift) with 10-bit target at 2^-24 */
        /* value = man * 2^(e-150); half subnormal unit = 2^-24 -> q = man * 2^(e-126) = man >> (126-e) */
        uint32_t q = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1u))) ++q;
        return (uint16_t)(sign | q);
    }
    uint32_t e = (absu >> 23) - 112u;
    uint32_t man = absu & 0x7FFFFFu;
    uint32_t q = (e << 10) | (man >> 13);
    uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) ++q; /* carry may bump the exponent: correct */
    return (uint16_t)(sign | q);
}

static inline float meta_to_f32(uint16_t bits, int meta) {
    return meta == ORC_META_F16 ? orc_f16_to_f32(bits) : orc_bf16_to_f32(bits);
}

/* -------------------------------------------------------------- blob layout */

void orc_expert_offsets(uint32_t d, uint32_t f, uint32_t bits, int additive_biases,
                        orc_offsets *o, uint64_t *stride_bytes) {
    uint64_t gate_weights = (uint64_t)f * d * bits / 8;
    uint64_t gate_meta = (uint64_t)f * (d / ORC_GROUP) * 2;
    uint64_t down_weights = (uint64_t)d * f * bits / 8;
    uint64_t down_meta = (uint64_t)d * (f / ORC_GROUP) * 2;
    uint64_t at = 0;
    o->gate_w = (uint32_t)at; at += gate_weights;
    o->gate_s = (uint32_t)at; at += gate_meta;
    o->gate_b = (uint32_t)at; at += gate_meta;
    o->up_w = (uint32_t)at; at += gate_weights;
    o->up_s = (uint32_t)at; at += gate_meta;
    o->up_b = (uint32_t)at; at += gate_meta;
    o->down_w = (uint32_t)at; at += down_weights;
    o->down_s = (uint32_t)at; at += down_meta;
    o->down_b = (uint32_t)at; at += down_meta;
    o->gate_ab = o->up_ab = o->down_ab = 0;
    if (additive_biases) {
        o->gate_ab = (uint32_t)at; at += (uint64_t)f * 2;
        o->up_ab = (uint32_t)at; at += (uint64_t)f * 2;
        o->down_ab = (uint32_t)at; at += (uint64_t)d * 2;
    }
    *stride_bytes = at;
}

/* -------------------------------------------------------------------- GEMVs */

void orc_int4_affine_gemv(const uint8_t *weights, const uint16_t *scales,
                          const uint16_t *biases, int meta, const float *x,
                          size_t rows, size_t n, float *out) {
    const size_t groups = n / ORC_GROUP;
    const size_t half_group = ORC_GROUP / 2;
    for (size_t r = 0; r < rows; ++r) {
        const uint8_t *row = weights + r * (n / 2);
        const uint16_t *srow = scales + r * groups;
        const uint16_t *brow = biases + r * groups;
        float total = 0.0f;
        for (size_t g = 0; g < groups; ++g) {
            const uint8_t *bytes = row + g * half_group;
            const float *xv = x + g * ORC_GROUP;
            float qx = 0.0f, xs = 0.0f;
            for (size_t k = 0; k < half_group; ++k) {
                const float even = xv[2 * k], odd = xv[2 * k + 1];
                const float lo = (float)(bytes[k] & 0x0F) * even;
                const float hi = (float)(bytes[k] >> 4) * odd;
                qx += lo + hi;
                xs += even + odd;
            }
            const float st = meta_to_f32(srow[g], meta) * qx;
            const float bt = meta_to_f32(brow[g], meta) * xs;
            total += st + bt;
        }
        out[r] = total;
    }
}

static inline uint32_t affine_q(const uint8_t *row, size_t element, int bits) {
    if (bits == 8) return row[element];
    const uint8_t byte = row[element >> 1];
    return (element & 1u) ? (uint32_t)(byte >> 4) : (uint32_t)(byte & 0x0F);
}

void orc_affine_gemv(const uint8_t *weights, const uint16_t *scales,
                     const uint16_t *biases, int meta, int bits, const float *x,
                     size_t rows, size_t n, float *out) {
    if (bits == 4) {
        orc_int4_affine_gemv(weights, scales, biases, meta, x, rows, n, out);
        return;
    }
    const size_t groups = n / ORC_GROUP;
    for (size_t r = 0; r < rows; ++r) {
        const uint8_t *row = weights + r * n;
        float total = 0.0f;
        for (size_t g = 0; g < groups; ++g) {
            float qx = 0.0f, xs = 0.0f;
            for (size_t k = 0; k < ORC_GROUP; k += 2) {
                const float even = x[g * ORC_GROUP + k], odd = x[g * ORC_GROUP + k + 1];
                const float lo = (float)row[g * ORC_GROUP + k] * even;
                const float hi = (float)row[g * ORC_GROUP + k + 1] * odd;
                qx += lo + hi;
                xs += even + odd;
            }
            const float st = meta_to_f32(scales[r * groups + g], meta) * qx;
            const float bt = meta_to_f32(biases[r * groups + g], meta) * xs;
            total += st + bt;
        }
        out[r] = total;
    }
}

void orc_affine_gemv_f64(const uint8_t *weights, const uint16_t *scales,
                         const uint16_t *biases, int meta, int bits, const float *x,
                         size_t rows, size_t n, double *out) {
    const size_t groups = n / ORC_GROUP;
    const size_t row_bytes = n * (size_t)bits / 8;
    for (size_t r = 0; r < rows; ++r) {
        const uint8_t *row = weights + r * row_bytes;
        double total = 0.0;
        for (size_t i = 0; i < n; ++i) {
            const size_t g = i / ORC_GROUP;
            const double w = (double)affine_q(row, i, bits) * (double)meta_to_f32(scales[r * groups + g], meta)
                + (double)meta_to_f32(biases[r * groups + g], meta);
            total += w * (double)x[i];
        }
        out[r] = total;
    }
}

/* -------------------------------------------------------------- activations */

static inline float silu_f(float v) { return v / (1.0f + expf(-v)); }

static inline float gelu_tanh_f(float v) {
    const float cube = v * v * v;
    float inner = 0.7978845608028654f * (v + 0.044715f * cube);
    if (inner < -20.0f) inner = -20.0f;
    if (inner > 20.0f) inner = 20.0f;
    return 0.5f * v * (1.0f + tanhf(inner));
}

float orc_glu(float gate, float up, int act) {
    if (act == ORC_ACT_CLAMPED_SWIGLU) {
        const float g = gate < 7.0f ? gate : 7.0f;
        float u = up;
        if (u < -7.0f) u = -7.0f;
        if (u > 7.0f) u = 7.0f;
        return (g / (1.0f + expf(-1.702f * g))) * (u + 1.0f);
    }
    return (act == ORC_ACT_SILU ? silu_f(gate) : gelu_tanh_f(gate)) * up;
}

/* --------------------------------------------------------------- CPU expert */

void orc_cpu_expert_ffn_accumulate(const uint8_t *expert, const orc_offsets *off,
                                   int meta, int bits, const float *x, uint32_t d,
                                   uint32_t f, float route_weight, float *scratch,
                                   float *out) {
    float *gate = scratch, *up = scratch + f, *down = scratch + 2 * (size_t)f;
    orc_affine_gemv(expert + off->gate_w, (const uint16_t *)(expert + off->gate_s),
                    (const uint16_t *)(expert + off->gate_b), meta, bits, x, f, d, gate);
    orc_affine_gemv(expert + off->up_w, (const uint16_t *)(expert + off->up_s),
                    (const uint16_t *)(expert + off->up_b), meta, bits, x, f, d, up);
    for (uint32_t i = 0; i < f; ++i) gate[i] = silu_f(gate[i]) * up[i];
    orc_affine_gemv(expert + off->down_w, (const uint16_t *)(expert + off->down_s),
                    (const uint16_t *)(expert + off->down_b), meta, bits, gate, d, f, down);
    for (uint32_t r = 0; r < d; ++r) out[r] += route_weight * down[r];
}

/* ------------------------------------------------------------ routed decode */

void orc_moe_phase1(const uint8_t *const *expert_base, const orc_offsets *off,
                    int meta, int bits, int act, int additive_biases,
                    const uint16_t *x_f16, uint32_t d, uint32_t f, uint32_t top_k,
                    uint16_t *acts_f16) {
    float *x = (float *)malloc(sizeof(float) * d);
    float *gate = (float *)malloc(sizeof(float) * f);
    float *up = (float *)malloc(sizeof(float) * f);
    for (uint32_t i = 0; i < d; ++i) x[i] = orc_f16_to_f32(x_f16[i]);
    for (uint32_t k = 0; k < top_k; ++k) {
        const uint8_t *base = expert_base[k];
        if (!base) continue; /* moe.metal:986 sentinel skip: acts keep their old value */
        orc_affine_gemv(base + off->gate_w, (const uint16_t *)(base + off->gate_s),
                        (const uint16_t *)(base + off->gate_b), meta, bits, x, f, d, gate);
        orc_affine_gemv(base + off->up_w, (const uint16_t *)(base + off->up_s),
                        (const uint16_t *)(base + off->up_b), meta, bits, x, f, d, up);
        for (uint32_t i = 0; i < f; ++i) {
            float g = gate[i], u = up[i];
            if (additive_biases) { /* moe.metal:261-269 */
                g += orc_bf16_to_f32(((const uint16_t *)(base + off->gate_ab))[i]);
                u += orc_bf16_to_f32(((const uint16_t *)(base + off->up_ab))[i]);
            }
            acts_f16[(size_t)k * f + i] = orc_f32_to_f16(orc_glu(g, u, act));
        }
    }
    free(x); free(gate); free(up);
}

void orc_moe_phase2(const uint8_t *const *expert_base, const orc_offsets *off,
                    int meta, int bits, int additive_biases,
                    const uint16_t *acts_f16, const uint16_t *routing_w_f16,
                    const uint16_t *residual_f16, uint32_t d, uint32_t f,
                    uint32_t top_k, uint16_t *y_f16, uint16_t *hidden_f16) {
    float *act = (float *)malloc(sizeof(float) * f);
    float *down = (float *)malloc(sizeof(float) * d);
    float *partial = (float *)calloc((size_t)top_k * d, sizeof(float));
    for (uint32_t k = 0; k < top_k; ++k) {
        const uint8_t *base = expert_base[k];
        if (!base) continue;
        for (uint32_t i = 0; i < f; ++i) act[i] = orc_f16_to_f32(acts_f16[(size_t)k * f + i]);
        orc_affine_gemv(base + off->down_w, (const uint16_t *)(base + off->down_s),
                        (const uint16_t *)(base + off->down_b), meta, bits, act, d, f, down);
        const float w = orc_f16_to_f32(routing_w_f16[k]);
        for (uint32_t r = 0; r < d; ++r) {
            float v = down[r];
            if (additive_biases) v += orc_bf16_to_f32(((const uint16_t *)(base + off->down_ab))[r]);
            partial[(size_t)k * d + r] = w * v; /* moe.metal:933 */
        }
    }
    for (uint32_t r = 0; r < d; ++r) {
        float acc = orc_f16_to_f32(residual_f16[r]); /* moe.metal:937-939 */
        for (uint32_t k = 0; k < top_k; ++k) acc += partial[(size_t)k * d + r];
        const uint16_t y = orc_f32_to_f16(acc);
        y_f16[r] = y;
        if (hidden_f16) { /* moe.metal:889-893 */
            hidden_f16[r] = orc_f32_to_f16(orc_f16_to_f32(hidden_f16[r]) + orc_f16_to_f32(y));
        }
    }
    free(act); free(down); free(partial);
}

/* ------------------------------------------------------------ shared expert */

void orc_shared_gate_up(const orc_proj *gate, const orc_proj *up, int meta, int bits,
                        const uint16_t *x_f16, uint32_t d, uint32_t f, uint16_t *gate_f16,
                        uint16_t *up_f16) {
    float *x = (float *)malloc(sizeof(float) * d);
    float *g = (float *)malloc(sizeof(float) * f);
    float *u = (float *)malloc(sizeof(float) * f);
    for (uint32_t i = 0; i < d; ++i) x[i] = orc_f16_to_f32(x_f16[i]);
    orc_affine_gemv(gate->w, gate->s, gate->b, meta, bits, x, f, d, g);
    orc_affine_gemv(up->w, up->s, up->b, meta, bits, x, f, d, u);
    for (uint32_t i = 0; i < f; ++i) { /* dequant_int4.metal:177-179: the GEMV writes half */
        gate_f16[i] = orc_f32_to_f16(g[i]);
        up_f16[i] = orc_f32_to_f16(u[i]);
    }
    free(x); free(g); free(u);
}

void orc_shared_down(const orc_proj *down, int meta, int bits, int act, const uint16_t *gate_f16,
                     const uint16_t *up_f16, uint32_t d, uint32_t f,
                     const uint16_t *scalar_gate_f16, uint16_t *h1_f16) {
    float *a = (float *)malloc(sizeof(float) * f);
    float *y = (float *)malloc(sizeof(float) * d);
    for (uint32_t i = 0; i < f; ++i) /* dequant_int4.metal:283-287; dequant_int8.metal:159-163 */
        a[i] = orc_f16_to_f32(orc_f32_to_f16(orc_glu(orc_f16_to_f32(gate_f16[i]), orc_f16_to_f32(up_f16[i]), act)));
    orc_affine_gemv(down->w, down->s, down->b, meta, bits, a, d, f, y);
    for (uint32_t r = 0; r < d; ++r) {
        uint16_t yh = orc_f32_to_f16(y[r]);
        if (scalar_gate_f16) { /* dequant_int4.metal:322-329 */
            const float sg = orc_f16_to_f32(scalar_gate_f16[0]);
            yh = orc_f32_to_f16(orc_f16_to_f32(yh) / (1.0f + expf(-sg)));
        }
        h1_f16[r] = yh;
    }
    free(a); free(y);
}

void orc_shared_expert(const orc_proj *gate, const orc_proj *up, const orc_proj *down,
                       int meta, int bits, int act, const uint16_t *x_f16, uint32_t d,
                       uint32_t f, const uint16_t *scalar_gate_f16, uint16_t *h1_f16) {
    uint16_t *g = (uint16_t *)malloc(sizeof(uint16_t) * f);
    uint16_t *u = (uint16_t *)malloc(sizeof(uint16_t) * f);
    orc_shared_gate_up(gate, up, meta, bits, x_f16, d, f, g, u);
    orc_shared_down(down, meta, bits, act, g, u, d, f, scalar_gate_f16, h1_f16);
    free(g); free(u);
}

/* shared_scalar_gate_rows, sources/Shrike/Metal/MoE/moe.metal:1154-1193: gate[row] = half(W . x_row)
 * for ONE 8-bit group-affine weight row against `rows` activation rows. Eight partial sums:
 * partial p takes the groups p, p+8, ... in order; inside a group lane l of 32 owns elements
 * 2l and 2l+1 (dot = q0*x0 + q1*x1, sum = x0 + x1; acc = fma(s, dot, acc); acc = fma(b, sum, acc));
 * the 32 lane sums are folded (the reference leaves the order to simd_sum; here the butterfly
 * v[l] += v[l^o], o = 1,2,4,8,16) and the eight partials are added in index order. */
void orc_shared_scalar_gate_rows(const uint8_t *w, const uint16_t *scales, const uint16_t *biases, int meta,
                                 const uint16_t *x_f16, uint32_t x_stride, uint32_t rows, uint32_t d,
                                 uint16_t *gate_f16) {
    const uint32_t groups = d / ORC_GROUP;
    for (uint32_t r = 0; r < rows; ++r) {
        const uint16_t *x = x_f16 + (size_t)r * x_stride;
        float total = 0.0f;
        for (uint32_t p = 0; p < 8; ++p) {
            float lane[32], next[32];
            for (uint32_t l = 0; l < 32; ++l) {
                float acc = 0.0f;
                for (uint32_t g = p; g < groups; g += 8) {
                    const uint32_t i0 = g * ORC_GROUP + 2 * l;
                    const float x0 = orc_f16_to_f32(x[i0]), x1 = orc_f16_to_f32(x[i0 + 1]);
                    const float q0 = (float)w[i0] * x0, q1 = (float)w[i0 + 1] * x1;
                    const float dot = q0 + q1, sum = x0 + x1;
                    acc = fmaf(meta_to_f32(scales[g], meta), dot, acc);
                    acc = fmaf(meta_to_f32(biases[g], meta), sum, acc);
                }
                lane[l] = acc;
            }
            for (uint32_t o = 1; o <= 16; o <<= 1) {
                for (uint32_t l = 0; l < 32; ++l) next[l] = lane[l] + lane[l ^ o];
                memcpy(lane, next, sizeof lane);
            }
            total += lane[0];
        }
        gate_f16[r] = orc_f32_to_f16(total);
    }
}

/* sigmoid_scalar_mul_rows_fp16, moe.metal:1195-1207: y[row, i] = half(y[row, i] / (1 + exp(-gate[row]))). */
void orc_sigmoid_scalar_mul_rows(uint16_t *y_f16, const uint16_t *gate_f16, uint32_t d, uint32_t rows) {
    for (uint32_t r = 0; r < rows; ++r) {
        const float g = orc_f16_to_f32(gate_f16[r]);
        for (uint32_t i = 0; i < d; ++i) {
            uint16_t *v = y_f16 + (size_t)r * d + i;
            *v = orc_f32_to_f16(orc_f16_to_f32(*v) / (1.0f + expf(-g)));
        }
    }
}

/* ------------------------------------------------------------------- router */

void orc_router_logits(const void *weights, const uint16_t *scales, const uint16_t *biases,
                       int router_kind, int meta, const uint16_t *hidden_f16,
                       const uint16_t *effective_scale_bf16, uint32_t num_experts,
                       uint32_t d, float *logits) {
    float *xs = (float *)malloc(sizeof(float) * d);
    for (uint32_t i = 0; i < d; ++i) /* moe.metal:357-358; the product is exact in fp32 */
        xs[i] = orc_f16_to_f32(hidden_f16[i]) * orc_bf16_to_f32(effective_scale_bf16[i]);
    const uint32_t elems_per_chunk = router_kind == ORC_ROUTER_F16 ? 8u
        : router_kind == ORC_ROUTER_AFFINE8 ? 16u : 32u;
    const uint32_t chunks = d / elems_per_chunk;
    const uint32_t groups = d / ORC_GROUP;
    for (uint32_t e = 0; e < num_experts; ++e) {
        float part[64];
        for (uint32_t l = 0; l < 64; ++l) {
            float acc = 0.0f;
            for (uint32_t c = l; c < chunks; c += 64) {
                const uint32_t first = c * elems_per_chunk;
                if (router_kind == ORC_ROUTER_F16) {
                    const uint16_t *row = (const uint16_t *)weights + (size_t)e * d;
                    for (uint32_t j = 0; j < 8; ++j)
                        acc = fmaf(orc_f16_to_f32(row[first + j]), xs[first + j], acc);
                } else {
                    const int bits = router_kind;
                    const uint8_t *row = (const uint8_t *)weights + (size_t)e * d * bits / 8;
                    float qx = 0.0f, sum = 0.0f;
                    for (uint32_t j = 0; j < elems_per_chunk; ++j) {
                        qx = fmaf((float)affine_q(row, first + j, bits), xs[first + j], qx);
                        sum = sum + xs[first + j];
                    }
                    const uint32_t g = first / ORC_GROUP;
                    acc = fmaf(meta_to_f32(scales[(size_t)e * groups + g], meta), qx, acc);
                    acc = fmaf(meta_to_f32(biases[(size_t)e * groups + g], meta), sum, acc);
                }
            }
            part[l] = acc;
        }
        for (uint32_t o = 32; o >= 1; o >>= 1) {
            float next[64];
            for (uint32_t l = 0; l < 64; ++l) next[l] = part[l] + part[l ^ o];
            memcpy(part, next, sizeof(part));
        }
        logits[e] = part[0];
    }
    free(xs);
}

static inline float sigmoid_f(float v) { return 1.0f / (1.0f + expf(-v)); }

void orc_router_select(const float *logits, const uint16_t *per_expert_scale_bf16,
                       const uint16_t *bias_bf16, uint32_t num_experts, uint32_t top_k,
                       int sigmoid_scores, float scaling, uint32_t *out_indices,
                       uint16_t *out_weights_f16) {
    uint32_t idx[8];
    float score[8];
    const uint32_t K = top_k < 8 ? top_k : 8;
    for (uint32_t i = 0; i < 8; ++i) { idx[i] = 0; score[i] = -INFINITY; }
    for (uint32_t e = 0; e < num_experts; ++e) {
        const float raw = logits[e];
        const float s = (sigmoid_scores ? sigmoid_f(raw) : raw) + orc_bf16_to_f32(bias_bf16[e]);
        if (s < score[K - 1]) continue;
        uint32_t pos = K;
        for (uint32_t i = 0; i < K; ++i) {
            if (s > score[i] || (s == score[i] && e < idx[i])) { pos = i; break; }
        }
        if (pos >= K) continue;
        for (uint32_t i = K - 1; i > pos; --i) { idx[i] = idx[i - 1]; score[i] = score[i - 1]; }
        idx[pos] = e;
        score[pos] = s;
    }
    if (sigmoid_scores) { /* moe.metal:460-474 */
        float orig[8], sum = 0.0f;
        for (uint32_t i = 0; i < K; ++i) { orig[i] = sigmoid_f(logits[idx[i]]); sum += orig[i]; }
        const float inv = scaling / (sum + 1e-20f);
        for (uint32_t i = 0; i < K; ++i) {
            out_indices[i] = idx[i];
            out_weights_f16[i] = orc_f32_to_f16(orig[i] * inv * orc_bf16_to_f32(per_expert_scale_bf16[idx[i]]));
        }
        return;
    }
    float ex[8], sum = 0.0f; /* moe.metal:477-490 */
    for (uint32_t i = 0; i < K; ++i) { ex[i] = expf(score[i] - score[0]); sum += ex[i]; }
    for (uint32_t i = 0; i < K; ++i) {
        out_indices[i] = idx[i];
        out_weights_f16[i] = orc_f32_to_f16((ex[i] / sum) * orc_bf16_to_f32(per_expert_scale_bf16[idx[i]]));
    }
}

uint32_t orc_classify(const uint32_t *topk, const uint64_t *residency, uint32_t top_k,
                      uint32_t num_experts, uint32_t *hit_count, uint32_t *hit_positions,
                      uint32_t *miss_count, uint32_t *miss_positions, uint32_t *miss_experts,
                      uint32_t *resolved_slots) {
    uint32_t hits = 0, misses = 0;
    for (uint32_t p = 0; p < top_k; ++p) {
        const uint32_t expert = topk[p] < num_experts - 1u ? topk[p] : num_experts - 1u;
        const uint64_t word = residency[expert];
        const uint32_t slot = (uint32_t)(word & 0xffffffffu), state = (uint32_t)(word >> 32);
        if (state == 2u && slot != 0xffffffffu) {
            hit_positions[hits++] = p;
            resolved_slots[p] = slot;
        } else {
            miss_positions[misses] = p;
            miss_experts[misses] = expert;
            ++misses;
            resolved_slots[p] = 0xffffffffu;
        }
    }
    hit_count[0] = hits;
    miss_count[0] = misses;
    return misses;
}

/* ------------------------------------------------------------------ prefill */

void orc_prefill_reduce(const uint16_t *partials_f16, const uint16_t *weights_f16,
                        uint32_t t, uint32_t top_k, uint32_t d, uint16_t *h2_f16) {
    for (uint32_t row = 0; row < t; ++row)
        for (uint32_t col = 0; col < d; ++col) {
            float acc = 0.0f;
            for (uint32_t r = 0; r < top_k; ++r)
                acc = fmaf(orc_f16_to_f32(weights_f16[(size_t)row * top_k + r]),
                           orc_f16_to_f32(partials_f16[((size_t)row * top_k + r) * d + col]), acc);
            h2_f16[(size_t)row * d + col] = orc_f32_to_f16(acc);
        }
}

void orc_residual_add_f16(uint16_t *hidden, const uint16_t *delta, size_t n) {
    for (size_t i = 0; i < n; ++i)
        hidden[i] = orc_f32_to_f16(orc_f16_to_f32(hidden[i]) + orc_f16_to_f32(delta[i]));
}

/* residual_add_rmsnorm_bf16w / rmsnorm_bf16w, sources/Shrike/Metal/Primitives/rmsnorm.metal:33-130:
 * hidden[i] = half(hidden[i] + delta[i]) in place (delta == NULL: no add), then
 * out[i] = half(hidden[i] * inv * weight[i]) with inv = 1/sqrt(mean(hidden^2) + eps) (mean and
 * reciprocal square root taken in fp64 from the fp32 sum, rounded to fp32 once), the sum of squares in fp32. The order of that sum is this build's own (the reference leaves it to
 * simd_sum): 256 threads, thread t takes the 8-element chunks t, t+256, ... with one fma chain,
 * each 64-lane wave folds with the xor butterfly 32...1, the four wave sums are added in order. */
void orc_residual_add_rmsnorm_bf16w(uint16_t *hidden, const uint16_t *delta, const uint16_t *weight_bf16,
                                    uint16_t *out, uint32_t d, float eps) {
    float acc[256];
    if (delta) orc_residual_add_f16(hidden, delta, d);
    for (uint32_t t = 0; t < 256; ++t) {
        float a = 0.0f;
        for (uint32_t c = t; c * 8u < d; c += 256u)
            for (uint32_t j = 0; j < 8u && c * 8u + j < d; ++j) {
                const float v = orc_f16_to_f32(hidden[c * 8u + j]);
                a = fmaf(v, v, a);
            }
        acc[t] = a;
    }
    float total = 0.0f;
    for (uint32_t w = 0; w < 4; ++w) {
        float lane[64], next[64];
        memcpy(lane, acc + 64u * w, sizeof lane);
        for (uint32_t o = 32; o >= 1; o >>= 1) {
            for (uint32_t l = 0; l < 64; ++l) next[l] = lane[l] + lane[l ^ o];
            memcpy(lane, next, sizeof lane);
        }
        total = w == 0 ? lane[0] : total + lane[0];
    }
    const float inv = (float)(1.0 / sqrt((double)total / (double)d + (double)eps));
    for (uint32_t i = 0; i < d; ++i)
        out[i] = orc_f32_to_f16(orc_f16_to_f32(hidden[i]) * inv * orc_bf16_to_f32(weight_bf16[i]));
}

/* -------------------------------------------------------- CPU layer (timing) */

typedef struct {
    const uint8_t *const *experts;
    const orc_offsets *off;
    int meta, bits;
    const float *x;
    uint32_t d, f, n_experts, first, step;
    float *down_all; /* [n_experts][d] */
} layer_task;

static void *layer_worker(void *arg) {
    layer_task *t = (layer_task *)arg;
    float *scratch = (float *)malloc(sizeof(float) * (2 * (size_t)t->f + t->d));
    for (uint32_t e = t->first; e < t->n_experts; e += t->step) {
        float *out = t->down_all + (size_t)e * t->d;
        memset(out, 0, sizeof(float) * t->d);
        orc_cpu_expert_ffn_accumulate(t->experts[e], t->off, t->meta, t->bits, t->x,
                                      t->d, t->f, 1.0f, scratch, out);
    }
    free(scratch);
    return NULL;
}

void orc_cpu_layer_fp32(const uint8_t *const *experts, const float *route_weights,
                        uint32_t n_experts, const orc_offsets *off, int meta, int bits,
                        const float *x, uint32_t d, uint32_t f, uint32_t threads, float *out) {
    if (threads < 1) threads = 1;
    if (threads > n_experts) threads = n_experts;
    float *down_all = (float *)malloc(sizeof(float) * (size_t)n_experts * d);
    pthread_t *tid = (pthread_t *)malloc(sizeof(pthread_t) * threads);
    layer_task *tasks = (layer_task *)malloc(sizeof(layer_task) * threads);
    for (uint32_t t = 0; t < threads; ++t) {
        tasks[t] = (layer_task){experts, off, meta, bits, x, d, f, n_experts, t, threads, down_all};
        if (t + 1 < threads) pthread_create(&tid[t], NULL, layer_worker, &tasks[t]);
    }
    layer_worker(&tasks[threads - 1]);
    for (uint32_t t = 0; t + 1 < threads; ++t) pthread_join(tid[t], NULL);
    for (uint32_t e = 0; e < n_experts; ++e)
        for (uint32_t r = 0; r < d; ++r) out[r] += route_weights[e] * down_all[(size_t)e * d + r];
    free(down_all); free(tid); free(tasks);
}
