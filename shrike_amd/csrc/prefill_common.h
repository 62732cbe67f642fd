// Shared between the prefill translation units: the device row-tile table that the
// grouping kernels write and the grouped FFN reads.
#pragma once

#include "gemv_common.h"

namespace shrike {

constexpr uint32_t kRowTile = 64;  // rows per row-tile entry (PrefillGroupedRoutedMoE.groupedRowTile)

// Worst case of row tiles for `pairs` pairs over `experts` experts: every expert may end
// in a partly filled tile.
inline uint32_t max_row_tiles(uint64_t pairs, uint32_t experts) {
    return uint32_t(pairs / kRowTile) + experts;
}

// fp16 halves of an fp32 value: hi + lo reproduces it to about 2^-22 relative
__device__ __forceinline__ uint32_t split_hi_lo(float v) {
    const uint16_t hi = f32_to_f16(v);
    const uint16_t lo = f32_to_f16(v - f16_to_f32(hi));
    return uint32_t(hi) | uint32_t(lo) << 16;
}

__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// Inclusive prefix sum over the lanes of a wave, lane 0 first.
__device__ __forceinline__ uint32_t wave_inclusive_scan_u32(uint32_t v, uint32_t lane) {
#pragma unroll
    for (uint32_t o = 1; o < 64u; o <<= 1) {
        const uint32_t below = __shfl_up(v, o);
        v += lane >= o ? below : 0u;
    }
    return v;
}

}  // namespace shrike
