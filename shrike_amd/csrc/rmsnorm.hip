// The step ahead of the router on decode: residual add and RMS norm in one launch
// (residual_add_rmsnorm_bf16w / rmsnorm_bf16w, sources/Shrike/Metal/Primitives/rmsnorm.metal:33-130),
// producing the fp16 row the router, the shared expert and phase 1 read. One workgroup a row.
#include "gemv_common.h"

namespace shrike {

// hidden[i] = half(hidden[i] + delta[i]) in place, then out[i] = half(hidden[i] * inv * weight[i])
// with inv = 1 / sqrt(mean(hidden^2) + eps). The sum of squares is fp32: thread t takes the
// 8-element chunks t, t+256, ... in one fma chain, a wave folds with the xor butterfly 32...1,
// the four wave sums are added in order; what follows the sum is taken in fp64 and rounded to
// fp32 once, so the row is reproducible bit for bit on a CPU.
__global__ __launch_bounds__(256) void k_residual_add_rmsnorm(uint16_t *hidden, const uint16_t *delta, const uint16_t *weight,
                                                              uint16_t *out, uint32_t d, float eps) {
    __shared__ float s_partial[4];
    uint16_t *row = hidden + size_t(blockIdx.x) * d;
    const uint16_t *delta_row = delta ? delta + size_t(blockIdx.x) * d : nullptr;
    uint16_t *out_row = out + size_t(blockIdx.x) * d;
    const uint32_t chunks = d / 8u;  // d is a multiple of 8
    constexpr int kMine = SHRIKE_MAX_HIDDEN / 8 / 256;  // chunks a thread can own
    uint4 mine[kMine];
    float acc = 0.0f;
#pragma unroll
    for (int r = 0; r < kMine; ++r) {
        const uint32_t c = threadIdx.x + 256u * r;
        if (c >= chunks) break;
        uint4 h = reinterpret_cast<const uint4 *>(row)[c];
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
            reinterpret_cast<uint4 *>(row)[c] = h;
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
        reinterpret_cast<uint4 *>(out_row)[c] = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

}  // namespace shrike

using namespace shrike;

extern "C" int shrike_hip_residual_add_rmsnorm_bf16w(void *stream, void *d_hidden, const void *d_delta, const void *d_weight,
                                                     void *d_out, uint32_t d, float eps, uint32_t rows) {
    SHRIKE_REQUIRE(d_hidden && d_weight && d_out, "rmsnorm: hidden, weight and out must be bound");
    SHRIKE_REQUIRE(d >= 8 && d % 8u == 0 && d <= SHRIKE_MAX_HIDDEN, "rmsnorm: d=%u must be a multiple of 8 up to %u", d,
                   SHRIKE_MAX_HIDDEN);
    SHRIKE_REQUIRE(((reinterpret_cast<uintptr_t>(d_hidden) | reinterpret_cast<uintptr_t>(d_delta) | reinterpret_cast<uintptr_t>(d_weight)
                     | reinterpret_cast<uintptr_t>(d_out)) & 15u) == 0,
                   "rmsnorm: buffers must be 16-byte aligned");
    SHRIKE_REQUIRE(rows <= 65535u * 1024u, "rmsnorm: %u rows is too many", rows);
    if (rows == 0) return 0;
    hipLaunchKernelGGL(k_residual_add_rmsnorm, dim3(rows), dim3(256), 0, as_stream(stream), static_cast<uint16_t *>(d_hidden),
                       static_cast<const uint16_t *>(d_delta), static_cast<const uint16_t *>(d_weight), static_cast<uint16_t *>(d_out),
                       d, eps);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}
