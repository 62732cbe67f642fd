// One row of residual add + RMS norm by a 256-thread workgroup, shared by the stand-alone kernel and
// by the head launch of the decode layer so that both produce the same bits
// (residual_add_rmsnorm_bf16w / rmsnorm_bf16w, sources/Shrike/Metal/Primitives/rmsnorm.metal:33-130).
#pragma once

#include "gemv_common.h"

namespace shrike {

// h[i] = half(hidden[i] + delta[i]) (delta may be null), out[i] = half(h[i] * inv * weight[i]) with
// inv = 1 / sqrt(mean(h^2) + eps). The sum of squares is fp32: thread t takes the 8-element chunks
// t, t+256, ... in one fma chain, a wave folds with the xor butterfly 32...1, the four wave sums are
// added in order; what follows the sum is taken in fp64 and rounded to fp32 once, so the row is
// reproducible bit for bit on a CPU. WRITE_HIDDEN stores h back over hidden. The normalised row goes
// to out_row (global, may be null) and to out_lds (may be null; a barrier follows, so every thread
// may read all of it on return). Every thread of the workgroup must call this.
template <bool WRITE_HIDDEN>
__device__ __forceinline__ void rmsnorm_row(uint16_t *hidden_row, const uint16_t *delta_row, const uint16_t *weight,
                                            uint16_t *out_row, uint4 *out_lds, uint32_t d, float eps, float (&s_partial)[4]) {
    const uint32_t chunks = d / 8u;  // d is a multiple of 8
    constexpr int kMine = SHRIKE_MAX_HIDDEN / 8 / 256;  // chunks a thread can own
    uint4 mine[kMine];
    float acc = 0.0f;
#pragma unroll
    for (int r = 0; r < kMine; ++r) {
        const uint32_t c = threadIdx.x + 256u * r;
        if (c >= chunks) break;
        uint4 h = reinterpret_cast<const uint4 *>(hidden_row)[c];
        uint32_t hw[4] = {h.x, h.y, h.z, h.w};
        if (delta_row) {
            const uint4 dl = reinterpret_cast<const uint4 *>(delta_row)[c];
            const uint32_t dw[4] = {dl.x, dl.y, dl.z, dl.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint16_t lo = f32_to_f16(__fadd_rn(f16_to_f32(uint16_t(hw[j])), f16_to_f32(uint16_t(dw[j]))));
                const uint16_t hi = f32_to_f16(__fadd_rn(f16_to_f32(uint16_t(hw[j] >> 16)), f16_to_f32(uint16_t(dw[j] >> 16))));
                hw[j] = uint32_t(lo) | uint32_t(hi) << 16;
            }
            h = make_uint4(hw[0], hw[1], hw[2], hw[3]);
            if (WRITE_HIDDEN) reinterpret_cast<uint4 *>(hidden_row)[c] = h;
        }
        mine[r] = h;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float lo = f16_to_f32(uint16_t(hw[j])), hi = f16_to_f32(uint16_t(hw[j] >> 16));
            acc = fmaf(lo, lo, acc);
            acc = fmaf(hi, hi, acc);
        }
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) acc = __fadd_rn(acc, __shfl_xor(acc, o));
    if ((threadIdx.x & 63u) == 0) s_partial[threadIdx.x >> 6] = acc;
    __syncthreads();
    const float total = __fadd_rn(__fadd_rn(__fadd_rn(s_partial[0], s_partial[1]), s_partial[2]), s_partial[3]);
    // the mean and the reciprocal square root in fp64, rounded to fp32 once: no dependence on how an
    // fp32 division or square root is expanded
    const float inv = float(1.0 / sqrt(double(total) / double(d) + double(eps)));
#pragma unroll
    for (int r = 0; r < kMine; ++r) {
        const uint32_t c = threadIdx.x + 256u * r;
        if (c >= chunks) break;
        const uint4 wv = reinterpret_cast<const uint4 *>(weight)[c];
        const uint32_t hw[4] = {mine[r].x, mine[r].y, mine[r].z, mine[r].w}, ww[4] = {wv.x, wv.y, wv.z, wv.w};
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float lo = __fmul_rn(__fmul_rn(f16_to_f32(uint16_t(hw[j])), inv), bf16_to_f32(uint16_t(ww[j])));
            const float hi = __fmul_rn(__fmul_rn(f16_to_f32(uint16_t(hw[j] >> 16)), inv), bf16_to_f32(uint16_t(ww[j] >> 16)));
            o[j] = uint32_t(f32_to_f16(lo)) | uint32_t(f32_to_f16(hi)) << 16;
        }
        const uint4 ov = make_uint4(o[0], o[1], o[2], o[3]);
        if (out_row) reinterpret_cast<uint4 *>(out_row)[c] = ov;
        if (out_lds) out_lds[c] = ov;
    }
    if (out_lds) __syncthreads();
}

}  // namespace shrike
