// The reference's CPU expert kernel behind its own C interface: shrike_int4_affine_gemv
// (sources/ShrikeKernelsC/include/shrike_kernels.h:9-29, sources/ShrikeKernelsC/int4_affine_gemv.c:28-135)
// and CPUExpertFFN.accumulate (sources/Shrike/Kernels/CPU/CPUExpertFFN.swift:102-140), which a runner uses
// for experts it keeps in host memory. Host-only: no device call, and nothing on the GPU path calls it.
//
// out[r] = sum_g ( scale[r][g] * sum_{i in g} q[r][i] x[i]  +  bias[r][g] * sum_{i in g} x[i] ), the two
// group sums running over element pairs in order: the rounding points of the reference's portable branch
// (int4_affine_gemv.c:114-134), so that the results are its bits. A byte's two codes are widened through a
// 256-entry table; the pair sums of x do not depend on the row and are formed once a call.
#include <cmath>
#include <cstring>
#include <vector>

#include "../../include/shrike_host.h"
#include "host_common.h"

namespace {

constexpr size_t kGroupElems = SHRIKE_GROUP_SIZE, kGroupBytes = kGroupElems / 2;

struct NibblePair {
    float lo, hi;
};
struct NibbleTable {
    NibblePair of[256];
    NibbleTable() {
        for (int b = 0; b < 256; ++b) of[b] = {float(b & 0x0F), float(b >> 4)};
    }
};
const NibbleTable g_codes;

inline float bf16(uint16_t bits) {
    const uint32_t u = uint32_t(bits) << 16;
    float v;
    std::memcpy(&v, &u, sizeof v);
    return v;
}

// sum_{pairs of the group, in order} (x_even + x_odd), one value a group; the same for every row
void group_sums_of(const float *x, size_t groups, float *out) {
    for (size_t g = 0; g < groups; ++g) {
        const float *xg = x + g * kGroupElems;
        float s = 0.0f;
        for (size_t k = 0; k < kGroupBytes; ++k) s += xg[2 * k] + xg[2 * k + 1];
        out[g] = s;
    }
}

void gemv_rows(const uint8_t *weights, const uint16_t *scales, const uint16_t *biases, const float *x, const float *xsum,
               size_t rows, size_t groups, float *out) {
    for (size_t r = 0; r < rows; ++r) {
        const uint8_t *codes = weights + r * groups * kGroupBytes;
        const uint16_t *s = scales + r * groups, *b = biases + r * groups;
        float acc = 0.0f;
        for (size_t g = 0; g < groups; ++g, codes += kGroupBytes) {
            const float *xg = x + g * kGroupElems;
            float dot = 0.0f;
            for (size_t k = 0; k < kGroupBytes; ++k) {
                const NibblePair q = g_codes.of[codes[k]];
                dot += q.lo * xg[2 * k] + q.hi * xg[2 * k + 1];
            }
            acc += bf16(s[g]) * dot + bf16(b[g]) * xsum[g];
        }
        out[r] = acc;
    }
}

inline float silu(float v) { return v / (1.0f + std::exp(-v)); }  // CPUExpertFFN.swift:92-94

}  // namespace

extern "C" {

void shrike_int4_affine_gemv(const uint8_t *weights, const uint16_t *scales, const uint16_t *biases, const float *x,
                             size_t rows, size_t n, float *out) {
    const size_t groups = n / kGroupElems;
    float stack_sums[64];
    std::vector<float> heap_sums;
    float *xsum = stack_sums;
    if (groups > 64) {
        heap_sums.resize(groups);
        xsum = heap_sums.data();
    }
    group_sums_of(x, groups, xsum);
    gemv_rows(weights, scales, biases, x, xsum, rows, groups, out);
}

size_t shrike_cpu_expert_ffn_scratch_floats(uint32_t d, uint32_t f) { return 2 * size_t(f) + size_t(d); }

int shrike_cpu_expert_ffn_accumulate(const void *expert, const shrike_expert_offsets *offsets, const float *x, uint32_t d,
                                     uint32_t f, float route_weight, float *scratch, float *out) {
    SHRIKE_REQUIRE(expert && offsets && x && scratch && out, "CPUExpertFFN.accumulate: NULL argument");
    SHRIKE_REQUIRE(d > 0 && f > 0 && d % kGroupElems == 0 && f % kGroupElems == 0,
                   "CPUExpertFFN.accumulate: d=%u and f=%u must be positive multiples of %u", d, f, SHRIKE_GROUP_SIZE);
    const uint8_t *base = static_cast<const uint8_t *>(expert);
    auto meta = [&](uint32_t off) { return reinterpret_cast<const uint16_t *>(base + off); };
    float *gate = scratch, *up = scratch + f, *down = scratch + 2 * size_t(f);
    // gate and up share x, and with it x's group sums (kept in the down rows' place until they are needed)
    float *xsum = down;
    group_sums_of(x, d / kGroupElems, xsum);
    gemv_rows(base + offsets->gate_w_off, meta(offsets->gate_s_off), meta(offsets->gate_b_off), x, xsum, f, d / kGroupElems, gate);
    gemv_rows(base + offsets->up_w_off, meta(offsets->up_s_off), meta(offsets->up_b_off), x, xsum, f, d / kGroupElems, up);
    for (uint32_t i = 0; i < f; ++i) gate[i] = silu(gate[i]) * up[i];
    // the activations' group sums go where `up` was
    group_sums_of(gate, f / kGroupElems, up);
    gemv_rows(base + offsets->down_w_off, meta(offsets->down_s_off), meta(offsets->down_b_off), gate, up, d, f / kGroupElems, down);
    for (uint32_t r = 0; r < d; ++r) out[r] += route_weight * down[r];
    return 0;
}

}  // extern "C"
