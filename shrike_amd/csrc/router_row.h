// The router's logit row, shared by the decode router and the prefill router so that both
// produce the same fp32 logits bit for bit.
#pragma once

#include "decode_launch.h"

namespace shrike {

// One expert row of the router GEMV (moe.metal:324-364), RK: 0 = fp16 rows, 8 / 4 =
// group-affine codes. The per-lane fused-multiply-add order and the xor butterfly are
// fixed so that the fp32 logits are reproducible bit for bit (lane l takes chunks
// l, l+64, ...).
// hidden, logits: the token's activation row and its logit row (a.hidden, a.logits_out for one token)
// x_source(): called once the row's own loads are in flight; returns the activation row to read (it may
// first have to produce it, e.g. a norm into LDS behind a barrier — then every wave of the workgroup
// must come through here or call it by itself). Returns the logit (in every lane).
// MAXI: 16-byte chunks a lane takes at most (chunks lane + 64 i, i < MAXI, past the row's end skipped); a row of up
// to 64 MAXI chunks gives the same sums under any larger MAXI, so a short row can run the narrower instance and
// leave out the loads of chunks it does not have.
template <int RK, int MAXI, class XSource>
__device__ __forceinline__ float router_row_n(const RouterArgs &a, XSource &&x_source, float *logits, uint32_t e, uint32_t lane,
                                              bool publish) {
    constexpr int E = RK == 0 ? 8 : RK == 8 ? 16 : 32;  // elements per 16-byte weight chunk
    constexpr int PIECES = E / 8;
    const uint32_t chunks = a.d / E;
    const uint32_t groups = a.d / kGroup;
    const uint32_t row_bytes = chunks * 16u;
    const uint8_t *row = static_cast<const uint8_t *>(a.weights) + size_t(e) * row_bytes;
    uint4 w[MAXI], xv[MAXI][PIECES], ev[MAXI][PIECES];
    uint16_t sc[MAXI], bi[MAXI];
#pragma unroll
    for (int i = 0; i < MAXI; ++i) {
        const uint32_t c = lane + 64u * i;
        const uint32_t cc = c < chunks ? c : 0u;
        w[i] = *reinterpret_cast<const uint4 *>(row + 16u * cc);
#pragma unroll
        for (int j = 0; j < PIECES; ++j) ev[i][j] = reinterpret_cast<const uint4 *>(a.effective_scale)[cc * PIECES + j];
        if (RK != 0) {
            sc[i] = a.scales[size_t(e) * groups + cc * E / kGroup];
            bi[i] = a.biases[size_t(e) * groups + cc * E / kGroup];
        }
    }
    const uint16_t *hidden = x_source();
#pragma unroll
    for (int i = 0; i < MAXI; ++i) {
        const uint32_t c = lane + 64u * i;
        const uint32_t cc = c < chunks ? c : 0u;
#pragma unroll
        for (int j = 0; j < PIECES; ++j) xv[i][j] = reinterpret_cast<const uint4 *>(hidden)[cc * PIECES + j];
    }
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < MAXI; ++i) {
        const uint32_t c = lane + 64u * i;
        if (c < chunks) {
            float xs[E];
#pragma unroll
            for (int j = 0; j < PIECES; ++j) {
                const uint32_t xw[4] = {xv[i][j].x, xv[i][j].y, xv[i][j].z, xv[i][j].w};
                const uint32_t ew[4] = {ev[i][j].x, ev[i][j].y, ev[i][j].z, ev[i][j].w};
#pragma unroll
                for (int t = 0; t < 4; ++t) {  // moe.metal:357-358 (exact product)
                    xs[8 * j + 2 * t] = __fmul_rn(f16_to_f32(uint16_t(xw[t])), bf16_to_f32(uint16_t(ew[t])));
                    xs[8 * j + 2 * t + 1] = __fmul_rn(f16_to_f32(uint16_t(xw[t] >> 16)), bf16_to_f32(uint16_t(ew[t] >> 16)));
                }
            }
            const uint32_t ww[4] = {w[i].x, w[i].y, w[i].z, w[i].w};
            if (RK == 0) {
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    acc = fmaf(f16_to_f32(uint16_t(ww[t])), xs[2 * t], acc);
                    acc = fmaf(f16_to_f32(uint16_t(ww[t] >> 16)), xs[2 * t + 1], acc);
                }
            } else {
                float qx = 0.0f, sum = 0.0f;
#pragma unroll
                for (int t = 0; t < E; ++t) {
                    const uint32_t q = RK == 8 ? (ww[t / 4] >> (8 * (t % 4))) & 0xffu
                                               : (ww[t / 8] >> (4 * (t % 8))) & 0xfu;
                    qx = fmaf(float(q), xs[t], qx);
                    sum = __fadd_rn(sum, xs[t]);
                }
                acc = fmaf(meta_f32(sc[i], a.meta), qx, acc);
                acc = fmaf(meta_f32(bi[i], a.meta), sum, acc);
            }
        }
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) acc = __fadd_rn(acc, __shfl_xor(acc, o));
    // publish: the logit is for another workgroup of the same launch and is written through to
    // device-coherent memory
    if (lane == 0) {
        if (publish) __hip_atomic_store(logits + e, acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else logits[e] = acc;
    }
    return acc;  // every lane holds the sum
}

template <int RK, class XSource>
__device__ __forceinline__ float router_row(const RouterArgs &a, XSource &&x_source, float *logits, uint32_t e, uint32_t lane,
                                            bool publish) {
    // fp16 rows: eight chunks a lane reach the activation ceiling (4,096); four cover hidden sizes up to 2,048
    if (RK == 0 && a.d <= 2048u) return router_row_n<RK, 4>(a, x_source, logits, e, lane, publish);
    return router_row_n<RK, RK == 0 ? 8 : 4>(a, x_source, logits, e, lane, publish);
}

template <int RK>
__device__ __forceinline__ float router_row(const RouterArgs &a, const uint16_t *hidden, float *logits, uint32_t e, uint32_t lane,
                                            bool publish) {
    return router_row<RK>(a, [&] { return hidden; }, logits, e, lane, publish);
}

template <int RK>
__device__ __forceinline__ float router_row(const RouterArgs &a, uint32_t e, uint32_t lane, bool publish = false) {
    return router_row<RK>(a, a.hidden, a.logits_out, e, lane, publish);
}

}  // namespace shrike
