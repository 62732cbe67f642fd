// The step ahead of the router on decode: residual add and RMS norm in one launch
// (residual_add_rmsnorm_bf16w / rmsnorm_bf16w, sources/Shrike/Metal/Primitives/rmsnorm.metal:33-130),
// producing the fp16 row the router, the shared expert and phase 1 read. One workgroup a row.
#include "rmsnorm_row.h"

namespace shrike {

// One workgroup a row; the arithmetic is rmsnorm_row's.
__global__ __launch_bounds__(256) void k_residual_add_rmsnorm(uint16_t *hidden, const uint16_t *delta, const uint16_t *weight,
                                                              uint16_t *out, uint32_t d, float eps) {
    __shared__ float s_partial[4];
    rmsnorm_row<true>(hidden + size_t(blockIdx.x) * d, delta ? delta + size_t(blockIdx.x) * d : nullptr, weight,
                      out + size_t(blockIdx.x) * d, nullptr, d, eps, s_partial);
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
