// Device helpers shared by the gfx950 kernels: 16-bit float decoding, wave64
// reductions over DPP, and the in-register dequant dot products.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

namespace shrike {

constexpr uint32_t kGroup = 64;
constexpr uint32_t kSentinel = 0xffffffffu;

typedef _Float16 h2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float(uint32_t(b) << 16); }
__device__ __forceinline__ float f16_to_f32(uint16_t b) {
    return float(__builtin_bit_cast(_Float16, b));
}
// Round-to-nearest-even of an fp32 value that has already been rounded to fp32. The empty
// asm keeps the compiler from folding a preceding multiply or fma into the conversion
// (v_fma_mixlo_f16), which rounds the unrounded result once and so differs from
// fp32-then-fp16 in about 6 of 100,000 values.
__device__ __forceinline__ uint16_t f32_to_f16(float v) {
    asm("" : "+v"(v));
    return __builtin_bit_cast(uint16_t, _Float16(v));
}
template <int META>
__device__ __forceinline__ float meta_to_f32(uint16_t b) {
    return META == 1 ? f16_to_f32(b) : bf16_to_f32(b);
}

__device__ __forceinline__ h2_t as_h2(uint32_t u) { return __builtin_bit_cast(h2_t, u); }
__device__ __forceinline__ uint32_t as_u32(h2_t h) { return __builtin_bit_cast(uint32_t, h); }

// ---- DPP lane exchange. Control codes: quad_perm = 0x00..0xff, row_mirror 0x140,
// row_half_mirror 0x141, row_bcast15 0x142, row_bcast31 0x143.
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xf, false));
}
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
    return uint32_t(__builtin_amdgcn_update_dpp(0, int(v), CTRL, ROW_MASK, 0xf, false));
}

// Sum over aligned lane segments of `seg` lanes (seg in {1,2,4,8,16,32,64}); every
// lane of a segment's last 16-lane row ends up holding the segment sum, and for
// seg <= 16 every lane of the segment does. Callers read lane (segment end - 1).
// A step that does not apply keeps v by a select, not by a branch: with a segment length known only at run time the
// six steps stay one straight run of instructions (a taken scalar branch a step costs more than the step).
__device__ __forceinline__ float seg_sum(float v, uint32_t seg) {
    float t;
    t = v + dpp_f32<0xB1>(v); v = seg >= 2 ? t : v;          // quad_perm [1,0,3,2]
    t = v + dpp_f32<0x4E>(v); v = seg >= 4 ? t : v;          // quad_perm [2,3,0,1]
    t = v + dpp_f32<0x141>(v); v = seg >= 8 ? t : v;         // row_half_mirror
    t = v + dpp_f32<0x140>(v); v = seg >= 16 ? t : v;        // row_mirror
    t = v + dpp_f32<0x142, 0xA>(v); v = seg >= 32 ? t : v;   // row_bcast15 into rows 1 and 3
    t = v + dpp_f32<0x143, 0xC>(v); v = seg >= 64 ? t : v;   // row_bcast31 into rows 2 and 3
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
    v = seg_sum(v, 64);
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// The wave's index in its workgroup, as a scalar: what is derived from it (rows, routed
// position, the cell and its base) then lives in scalar registers and scalar loads.
__device__ __forceinline__ uint32_t wave_index() { return uint32_t(__builtin_amdgcn_readfirstlane(int(threadIdx.x >> 6))); }

// Every store this wave has issued is complete; for a write-through (device-scope atomic)
// store that means visible device-wide. Cheaper than a device-scope release fence, which
// also writes back the whole second-level cache of this group of compute units.
__device__ __forceinline__ void wait_stores() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Wave-wide float max / unsigned min, broadcast to every lane. Rows a step does not
// write keep their own value (old = self), so the partial results stay valid operands.
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_keep_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, ROW_MASK, 0xf, false));
}
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ uint32_t dpp_keep_u32(uint32_t v) {
    return uint32_t(__builtin_amdgcn_update_dpp(int(v), int(v), CTRL, ROW_MASK, 0xf, false));
}
__device__ __forceinline__ float wave_max_f32(float v) {
    v = fmaxf(v, dpp_keep_f32<0xB1>(v));
    v = fmaxf(v, dpp_keep_f32<0x4E>(v));
    v = fmaxf(v, dpp_keep_f32<0x141>(v));
    v = fmaxf(v, dpp_keep_f32<0x140>(v));
    v = fmaxf(v, dpp_keep_f32<0x142, 0xA>(v));
    v = fmaxf(v, dpp_keep_f32<0x143, 0xC>(v));
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
// Written out in assembly so that each step is one DPP-fused max (rows a step's row mask
// leaves out keep their value); a DPP read of a register needs two wait states after the
// write before it.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    asm volatile(
        "s_nop 1\n\t"
        "v_max_u32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_u32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_u32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_u32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_u32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_u32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
        "s_nop 1"
        : "+v"(v));
    return uint32_t(__builtin_amdgcn_readlane(int(v), 63));
}
__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) {
    v = min(v, dpp_keep_u32<0xB1>(v));
    v = min(v, dpp_keep_u32<0x4E>(v));
    v = min(v, dpp_keep_u32<0x141>(v));
    v = min(v, dpp_keep_u32<0x140>(v));
    v = min(v, dpp_keep_u32<0x142, 0xA>(v));
    v = min(v, dpp_keep_u32<0x143, 0xC>(v));
    return uint32_t(__builtin_amdgcn_readlane(int(v), 63));
}

// Max of a 64-bit key over the wave; result broadcast to every lane.
__device__ __forceinline__ uint64_t wave_max_u64(uint64_t key) {
    uint32_t lo = uint32_t(key), hi = uint32_t(key >> 32);
#define SHRIKE_MAX_STEP(CTRL, MASK)                                             \
    {                                                                            \
        const uint32_t olo = dpp_u32<CTRL, MASK>(lo), ohi = dpp_u32<CTRL, MASK>(hi); \
        const bool take = ohi > hi || (ohi == hi && olo > lo);                  \
        lo = take ? olo : lo;                                                   \
        hi = take ? ohi : hi;                                                   \
    }
    SHRIKE_MAX_STEP(0xB1, 0xf)
    SHRIKE_MAX_STEP(0x4E, 0xf)
    SHRIKE_MAX_STEP(0x141, 0xf)
    SHRIKE_MAX_STEP(0x140, 0xf)
    SHRIKE_MAX_STEP(0x142, 0xA)
    SHRIKE_MAX_STEP(0x143, 0xC)
#undef SHRIKE_MAX_STEP
    lo = uint32_t(__builtin_amdgcn_readlane(int(lo), 63));
    hi = uint32_t(__builtin_amdgcn_readlane(int(hi), 63));
    return (uint64_t(hi) << 32) | lo;
}

// ---- 16-byte chunk of codes against the lane's activation slice.
//
// A chunk is 4 little-endian words. For 4-bit codes word j holds elements 8j..8j+7
// (element i in bits 4i..4i+3). A code needs no conversion to enter the fp16 dot: the
// bit pattern 0x000q is the fp16 subnormal q * 2^-24 and 0x00q0 is q * 2^-20, both exact,
// and the 2-way fp16 dot of gfx950 takes subnormal inputs at full precision (products are
// exact in fp32, the sum is kept in fp32). So (w & 0x000F000F) is the pair {q0, q4} * 2^-24
// and (w & 0x00F000F0) the pair {q1, q5} * 2^-20; after one shift by 8 the same two masks
// give {q2, q6} and {q3, q7}. The two scalings go to two accumulators that are joined once
// per chunk: dot = (lo * 16 + hi) * 2^20. The activation slice is therefore kept as the
// pairs (e0,e4) (e1,e5) (e2,e6) (e3,e7) per word (pairs_from_x8 below).
struct XChunk4 { h2_t p[16]; };   // 32 activations of a 4-bit chunk, pair layout
struct XChunk8 { h2_t p[8]; };    // 16 activations of an 8-bit chunk, natural pairs

__device__ __forceinline__ void pairs_from_x8(const uint4 v, h2_t *p) {
    // v = elements e0..e7 as (e0,e1)(e2,e3)(e4,e5)(e6,e7)
    p[0] = as_h2(__builtin_amdgcn_perm(v.z, v.x, 0x05040100u));  // (e0,e4)
    p[1] = as_h2(__builtin_amdgcn_perm(v.z, v.x, 0x07060302u));  // (e1,e5)
    p[2] = as_h2(__builtin_amdgcn_perm(v.w, v.y, 0x05040100u));  // (e2,e6)
    p[3] = as_h2(__builtin_amdgcn_perm(v.w, v.y, 0x07060302u));  // (e3,e7)
}

// The first dot of a chain, against a zero accumulator. The compiler only forms the two-operand dot (the accumulator is
// the destination) and would clear a register for every chain first; the three-operand form takes the zero as a constant.
__device__ __forceinline__ float dot2_from_zero(h2_t a, h2_t b) {
    float r;
    asm("v_dot2_f32_f16 %0, %1, %2, 0" : "=v"(r) : "v"(a), "v"(b));
    return r;
}

// fp32 sum of 8 fp16 activations: four 2-way dots against (1, 1).
__device__ __forceinline__ float sum_x8(const uint4 v) {
    const h2_t one = {(_Float16)1.0f, (_Float16)1.0f};
    float s = dot2_from_zero(as_h2(v.x), one);
    s = __builtin_amdgcn_fdot2(as_h2(v.y), one, s, false);
    s = __builtin_amdgcn_fdot2(as_h2(v.z), one, s, false);
    s = __builtin_amdgcn_fdot2(as_h2(v.w), one, s, false);
    return s;
}

__device__ __forceinline__ void dot_word4(uint32_t w, const h2_t *p, float &lo, float &hi) {
    const uint32_t w8 = w >> 8;
    lo = __builtin_amdgcn_fdot2(as_h2(w & 0x000F000Fu), p[0], lo, false);
    hi = __builtin_amdgcn_fdot2(as_h2(w & 0x00F000F0u), p[1], hi, false);
    lo = __builtin_amdgcn_fdot2(as_h2(w8 & 0x000F000Fu), p[2], lo, false);
    hi = __builtin_amdgcn_fdot2(as_h2(w8 & 0x00F000F0u), p[3], hi, false);
}

// the same for the first word of a chunk: its first two dots start the two accumulators
__device__ __forceinline__ void dot_word4_first(uint32_t w, const h2_t *p, float &lo, float &hi) {
    const uint32_t w8 = w >> 8;
    lo = dot2_from_zero(as_h2(w & 0x000F000Fu), p[0]);
    hi = dot2_from_zero(as_h2(w & 0x00F000F0u), p[1]);
    lo = __builtin_amdgcn_fdot2(as_h2(w8 & 0x000F000Fu), p[2], lo, false);
    hi = __builtin_amdgcn_fdot2(as_h2(w8 & 0x00F000F0u), p[3], hi, false);
}

__device__ __forceinline__ float dot_chunk4(const uint4 w, const XChunk4 &x) {
    float lo, hi;
    dot_word4_first(w.x, x.p + 0, lo, hi);
    dot_word4(w.y, x.p + 4, lo, hi);
    dot_word4(w.z, x.p + 8, lo, hi);
    dot_word4(w.w, x.p + 12, lo, hi);
    return fmaf(lo, 16.0f, hi) * 1048576.0f;
}

// 8-bit codes: bytes b0..b3 of a word are elements 4j..4j+3; a byte permute spreads two
// of them over the low bytes of the two halves: {b0, b1} * 2^-24 as fp16 subnormals.
__device__ __forceinline__ float dot_word8(uint32_t w, const h2_t *p, float acc) {
    acc = __builtin_amdgcn_fdot2(as_h2(__builtin_amdgcn_perm(0u, w, 0x0c010c00u)), p[0], acc, false);
    acc = __builtin_amdgcn_fdot2(as_h2(__builtin_amdgcn_perm(0u, w, 0x0c030c02u)), p[1], acc, false);
    return acc;
}

__device__ __forceinline__ float dot_chunk8(const uint4 w, const XChunk8 &x) {
    float acc = dot2_from_zero(as_h2(__builtin_amdgcn_perm(0u, w.x, 0x0c010c00u)), x.p[0]);
    acc = __builtin_amdgcn_fdot2(as_h2(__builtin_amdgcn_perm(0u, w.x, 0x0c030c02u)), x.p[1], acc, false);
    acc = dot_word8(w.y, x.p + 2, acc);
    acc = dot_word8(w.z, x.p + 4, acc);
    acc = dot_word8(w.w, x.p + 6, acc);
    return acc * 16777216.0f;
}

__device__ __forceinline__ float silu(float v) { return v / (1.0f + expf(-v)); }
__device__ __forceinline__ float gelu_tanh(float v) {
    const float cube = v * v * v;
    float inner = 0.7978845608028654f * (v + 0.044715f * cube);
    inner = fminf(fmaxf(inner, -20.0f), 20.0f);
    return 0.5f * v * (1.0f + tanhf(inner));
}
// The same three activations through the hardware's exp2 and reciprocal (each within 1 ulp of fp32; a sigmoid
// a few ulp): for results that are rounded to fp16 next, where a correctly rounded division and expf buy nothing.
// gelu_tanh(v) = v * sigmoid(2 * inner), since 0.5 * (1 + tanh(t)) = 1 / (1 + exp(-2 t)).
__device__ __forceinline__ float sigmoid_fast(float v) {
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * v));
}
template <int ACT>
__device__ __forceinline__ float glu_fast(float gate, float up) {
    if (ACT == 2) {
        const float g = fminf(gate, 7.0f);
        const float u = fminf(fmaxf(up, -7.0f), 7.0f);
        return (g * sigmoid_fast(1.702f * g)) * (u + 1.0f);
    }
    if (ACT == 1) return (gate * sigmoid_fast(gate)) * up;
    const float cube = gate * gate * gate;
    float inner = 0.7978845608028654f * (gate + 0.044715f * cube);
    inner = fminf(fmaxf(inner, -20.0f), 20.0f);
    return (gate * sigmoid_fast(2.0f * inner)) * up;
}

// moe.metal:280-288
template <int ACT>
__device__ __forceinline__ float glu(float gate, float up) {
    if (ACT == 2) {
        const float g = fminf(gate, 7.0f);
        const float u = fminf(fmaxf(up, -7.0f), 7.0f);
        return (g / (1.0f + expf(-1.702f * g))) * (u + 1.0f);
    }
    return (ACT == 1 ? silu(gate) : gelu_tanh(gate)) * up;
}


// A kernel's by-value argument block sits in constant memory and the compiler fetches its fields where
// they are first used, each first touch of a 64-byte line a miss of the scalar cache on the way to the
// first useful load. One dword of every line, requested together at the kernel's start, turns those
// misses into one.
template <typename Args>
__device__ __forceinline__ void warm_kernel_arguments(const Args &a) {
    const uint32_t *words = reinterpret_cast<const uint32_t *>(&a);
    constexpr uint32_t lines = (sizeof(Args) + 63u) / 64u;
    uint32_t touched[lines];
#pragma unroll
    for (uint32_t i = 0; i < lines; ++i) touched[i] = __builtin_nontemporal_load(words + (i * 16u < sizeof(Args) / 4u ? i * 16u : sizeof(Args) / 4u - 1u));
#pragma unroll
    for (uint32_t i = 0; i < lines; ++i) asm volatile("" ::"s"(touched[i]));
}
}  // namespace shrike
