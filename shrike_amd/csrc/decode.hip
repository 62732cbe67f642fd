// Decode-time routed-expert kernels for gfx950 and their C-ABI entry points:
// router GEMV + top-k select (+ residency classify), phase 1 (gate/up matvec +
// GLU), phase 2 (down matvec + weighted combine + residual), and the dense
// group-affine GEMV the shared expert is made of.
//
// Shape of every matvec here: a row of codes is a run of 16-byte chunks; lane l of
// a 64-wide wave owns column chunks l, l+64, ... of every row it touches, so its
// slice of the activation vector sits in registers once (already in the pair
// layout the fp16 dot wants) and each row costs one 128-bit load per chunk. The
// kernels are HBM-bound: all of a wave's row loads are issued before the first is
// consumed, and out-of-range chunks are clamped to a valid address and zeroed
// rather than predicated, so the loads stay back to back.
#include "device_utils.h"
#include "host_common.h"

namespace shrike {

struct PoolArg {
    const uint8_t *base[SHRIKE_POOL_MAX_CHUNKS];
    uint32_t cells_per_chunk;
};

// moe.metal:302-305
__device__ __forceinline__ const uint8_t *cell_base(const PoolArg &pool, uint32_t cell, uint64_t stride) {
    return pool.base[cell / pool.cells_per_chunk] + uint64_t(cell % pool.cells_per_chunk) * stride;
}

__device__ __forceinline__ float meta_f32(uint16_t b, uint32_t meta) {
    return meta == SHRIKE_META_F16 ? f16_to_f32(b) : bf16_to_f32(b);
}

__device__ __forceinline__ float glu_rt(float g, float u, uint32_t act) {
    return act == SHRIKE_ACT_CLAMPED_SWIGLU ? glu<2>(g, u) : act == SHRIKE_ACT_SILU ? glu<1>(g, u) : glu<0>(g, u);
}

// moe.metal:36-39
__device__ __forceinline__ bool io_ready(const uint32_t *io_status) {
    if (!io_status) return true;
    const uint32_t st = io_status[0];
    return st == 1u || st == 3u;
}

template <int BITS> struct Chunk;
template <> struct Chunk<4> {
    static constexpr int E = 32, PIECES = 4;
    typedef XChunk4 X;
    static __device__ __forceinline__ void fill(X &x, int piece, const uint4 v) { pairs_from_x8(v, x.p + 4 * piece); }
    static __device__ __forceinline__ float dot(const uint4 w, const X &x) { return dot_chunk4(w, x); }
};
template <> struct Chunk<8> {
    static constexpr int E = 16, PIECES = 2;
    typedef XChunk8 X;
    static __device__ __forceinline__ void fill(X &x, int piece, const uint4 v) {
        x.p[4 * piece + 0] = as_h2(v.x);
        x.p[4 * piece + 1] = as_h2(v.y);
        x.p[4 * piece + 2] = as_h2(v.z);
        x.p[4 * piece + 3] = as_h2(v.w);
    }
    static __device__ __forceinline__ float dot(const uint4 w, const X &x) { return dot_chunk8(w, x); }
};

__device__ __forceinline__ uint4 zero4() { return make_uint4(0u, 0u, 0u, 0u); }

// The lane's activation slices for column chunks col + 64*i, read as 16-byte pieces
// from `vec` (global or LDS), with the fp32 sum of each slice for the bias term.
template <int BITS, int NCH>
__device__ __forceinline__ void load_slices(const uint4 *vec, uint32_t cpr, uint32_t col, bool lane_on,
                                            typename Chunk<BITS>::X (&x)[NCH], float (&xs)[NCH]) {
    typedef Chunk<BITS> C;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const uint32_t c = col + 64u * i;
        const bool on = lane_on && c < cpr;
        const uint32_t cc = on ? c : 0u;
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < C::PIECES; ++j) {
            uint4 v = vec[cc * C::PIECES + j];
            if (!on) v = zero4();
            C::fill(x[i], j, v);
            s += sum_x8(v);
        }
        xs[i] = s;
    }
}

// One row's codes and metadata for the lane's column chunks.
template <int BITS, int NCH>
struct RowRegs {
    uint4 w[NCH];
    uint16_t s[NCH], b[NCH];
};

template <int BITS, int NCH>
__device__ __forceinline__ void load_row(RowRegs<BITS, NCH> &r, const uint8_t *w_row, const uint16_t *s_row,
                                         const uint16_t *b_row, uint32_t cpr, uint32_t col, bool lane_on) {
    typedef Chunk<BITS> C;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const uint32_t c = col + 64u * i;
        const bool on = lane_on && c < cpr;
        const uint32_t cc = on ? c : 0u;
        const uint32_t g = cc * C::E / kGroup;
        uint4 w = *reinterpret_cast<const uint4 *>(w_row + 16u * cc);
        uint16_t s = s_row[g], b = b_row[g];
        if (!on) { w = zero4(); s = 0; b = 0; }
        r.w[i] = w; r.s[i] = s; r.b[i] = b;
    }
}

template <int BITS, int NCH>
__device__ __forceinline__ float row_partial(const RowRegs<BITS, NCH> &r, const typename Chunk<BITS>::X (&x)[NCH],
                                             const float (&xs)[NCH], uint32_t meta) {
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        acc = fmaf(meta_f32(r.s[i], meta), Chunk<BITS>::dot(r.w[i], x[i]), acc);
        acc = fmaf(meta_f32(r.b[i], meta), xs[i], acc);
    }
    return acc;
}

// ------------------------------------------------------------------- router

struct RouterArgs {
    const void *weights;
    const uint16_t *scales, *biases;
    const uint16_t *hidden, *effective_scale, *per_expert_scale, *logit_bias;
    float *logits;
    uint32_t *counter;
    uint32_t *out_indices;
    uint16_t *out_weights;
    uint32_t num_experts, d, top_k, meta, sigmoid;
    float scaling;
    // classify (residency == nullptr: router only)
    const uint64_t *residency;
    uint32_t *hit_count, *hit_positions, *miss_count, *miss_positions, *miss_experts, *resolved_slots;
};

__device__ __forceinline__ uint32_t orderable(float v) {
    const uint32_t u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float from_orderable(uint32_t o) {
    return __uint_as_float((o & 0x80000000u) ? (o & 0x7fffffffu) : ~o);
}
__device__ __forceinline__ float sigmoidf_(float v) { return 1.0f / (1.0f + expf(-v)); }
__device__ __forceinline__ float load_coherent(const float *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// moe.metal:419-491, run by one wave: lane l holds experts l, l+64, l+128, l+192;
// top_k rounds of a wave-wide max over the key (orderable score, then lower index).
__device__ uint32_t select_wave(const RouterArgs &a, uint32_t lane) {
    uint64_t key[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t e = lane + 64u * j;
        key[j] = 0;
        if (e < a.num_experts) {
            const float raw = load_coherent(a.logits + e);
            float s = (a.sigmoid ? sigmoidf_(raw) : raw) + bf16_to_f32(a.logit_bias[e]);
            s = s + 0.0f;  // -0 and +0 tie
            if (s == s) key[j] = (uint64_t(orderable(s)) << 32) | uint64_t(0xffffffffu - e);
        }
    }
    uint32_t idx[8];
    float score[8];
    const uint32_t K = a.top_k;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        idx[r] = 0; score[r] = -INFINITY;
        if (uint32_t(r) < K) {
            uint64_t best = key[0];
#pragma unroll
            for (int j = 1; j < 4; ++j) best = key[j] > best ? key[j] : best;
            const uint64_t win = wave_max_u64(best);
            if (win != 0) {
                idx[r] = 0xffffffffu - uint32_t(win);
                score[r] = from_orderable(uint32_t(win >> 32));
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) key[j] = key[j] == win ? 0 : key[j];
        }
    }
    float w[8];
    if (a.sigmoid) {  // moe.metal:460-474
        float sum = 0.0f;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            w[r] = uint32_t(r) < K ? sigmoidf_(load_coherent(a.logits + idx[r])) : 0.0f;
            if (uint32_t(r) < K) sum += w[r];
        }
        const float inv = a.scaling / (sum + 1e-20f);
#pragma unroll
        for (int r = 0; r < 8; ++r) w[r] = w[r] * inv;
    } else {  // moe.metal:477-490
        float sum = 0.0f;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            w[r] = uint32_t(r) < K ? expf(score[r] - score[0]) : 0.0f;
            if (uint32_t(r) < K) sum += w[r];
        }
#pragma unroll
        for (int r = 0; r < 8; ++r) w[r] = w[r] / sum;
    }
    uint32_t mine = 0;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        if (lane == uint32_t(r) && uint32_t(r) < K) {
            a.out_indices[r] = idx[r];
            a.out_weights[r] = f32_to_f16(w[r] * bf16_to_f32(a.per_expert_scale[idx[r]]));
            mine = idx[r];
        }
    }
    return mine;  // lane p < top_k: the expert at position p
}

// moe.metal:121-151, one wave; lane p classifies position p.
__device__ void classify_wave(uint32_t my_expert, const uint64_t *residency, uint32_t top_k,
                              uint32_t num_experts, uint32_t lane, uint32_t *hit_count,
                              uint32_t *hit_positions, uint32_t *miss_count, uint32_t *miss_positions,
                              uint32_t *miss_experts, uint32_t *resolved_slots, uint32_t *out_misses) {
    const bool on = lane < top_k;
    uint32_t expert = 0, slot = kSentinel, state = 0;
    if (on) {
        expert = min(my_expert, num_experts - 1u);
        const uint64_t word = residency[expert];
        slot = uint32_t(word);
        state = uint32_t(word >> 32);
    }
    const bool hit = on && state == SHRIKE_RESIDENCY_RESIDENT && slot != kSentinel;
    const uint64_t hit_mask = __ballot(hit), miss_mask = __ballot(on && !hit);
    const uint64_t below = (uint64_t(1) << lane) - 1u;
    if (hit) {
        hit_positions[__popcll(hit_mask & below)] = lane;
        resolved_slots[lane] = slot;
    } else if (on) {
        const uint32_t at = __popcll(miss_mask & below);
        miss_positions[at] = lane;
        miss_experts[at] = expert;
        resolved_slots[lane] = kSentinel;
    }
    if (lane == 0) {
        hit_count[0] = __popcll(hit_mask);
        miss_count[0] = __popcll(miss_mask);
    }
    *out_misses = __popcll(miss_mask);
}

// RK: 0 = fp16 rows, 8 / 4 = group-affine codes. One wave per expert row; the
// per-lane fused-multiply-add order and the xor butterfly are fixed so that the
// fp32 logits are reproducible bit for bit (lane l takes chunks l, l+64, ...).
template <int RK>
__global__ __launch_bounds__(256) void k_router(RouterArgs a) {
    constexpr int E = RK == 0 ? 8 : RK == 8 ? 16 : 32;  // elements per 16-byte weight chunk
    constexpr int PIECES = E / 8;
    constexpr int MAXI = RK == 0 ? 8 : 4;
    __shared__ uint32_t s_last;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t e = blockIdx.x * 4u + wave;
    const uint32_t chunks = a.d / E;
    const uint32_t groups = a.d / kGroup;
    if (e < a.num_experts) {
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
            for (int j = 0; j < PIECES; ++j) {
                xv[i][j] = reinterpret_cast<const uint4 *>(a.hidden)[cc * PIECES + j];
                ev[i][j] = reinterpret_cast<const uint4 *>(a.effective_scale)[cc * PIECES + j];
            }
            if (RK != 0) {
                sc[i] = a.scales[size_t(e) * groups + cc * E / kGroup];
                bi[i] = a.biases[size_t(e) * groups + cc * E / kGroup];
            }
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
        if (lane == 0) {
            a.logits[e] = acc;
            __threadfence();
        }
    }
    if (!a.out_indices) return;  // scores only
    __syncthreads();
    if (threadIdx.x == 0) {
        __threadfence();
        s_last = atomicAdd(a.counter, 1u) == gridDim.x - 1u ? 1u : 0u;
    }
    __syncthreads();
    if (!s_last || wave != 0) return;
    __threadfence();
    const uint32_t mine = select_wave(a, lane);
    if (a.residency) {
        uint32_t misses;
        classify_wave(mine, a.residency, a.top_k, a.num_experts, lane, a.hit_count, a.hit_positions,
                      a.miss_count, a.miss_positions, a.miss_experts, a.resolved_slots, &misses);
    }
    if (lane == 0) *a.counter = 0u;
}

struct ClassifyArgs {
    const uint32_t *topk;
    const uint64_t *residency;
    uint32_t *hit_count, *hit_positions, *miss_count, *miss_positions, *miss_experts, *resolved_slots;
    uint32_t top_k, num_experts;
    uint32_t full_grids[12];
    uint32_t *spec_args;
    uint32_t *host_readback;
    uint32_t tag;
    const uint16_t *topk_weights;
    const uint32_t *predicted;
};

// moe.metal:194-231 with the readback of :158-181.
__global__ __launch_bounds__(64) void k_classify(ClassifyArgs a) {
    const uint32_t lane = threadIdx.x;
    uint32_t misses;
    classify_wave(lane < a.top_k ? a.topk[lane] : 0u, a.residency, a.top_k, a.num_experts, lane, a.hit_count, a.hit_positions,
                  a.miss_count, a.miss_positions, a.miss_experts, a.resolved_slots, &misses);
    const bool all_hit = misses == 0u;
    if (a.spec_args && lane < 3) {
        const uint32_t zero_grid = lane == 0 ? 0u : 1u;
        a.spec_args[lane] = a.full_grids[lane];
        a.spec_args[3 + lane] = all_hit ? a.full_grids[3 + lane] : zero_grid;
        a.spec_args[6 + lane] = all_hit ? zero_grid : a.full_grids[6 + lane];
        a.spec_args[9 + lane] = all_hit ? zero_grid : a.full_grids[9 + lane];
    }
    if (a.tag != 0u && a.host_readback) {
        __threadfence_block();
        __syncthreads();  // positions written above by other lanes
        const uint32_t hits = a.top_k - misses, t = a.tag << 16, K = a.top_k;
        if (lane == 0) {
            a.host_readback[0] = t | hits;
            a.host_readback[1] = t | misses;
        }
        if (lane < K) {
            a.host_readback[2 + lane] = t | min(a.topk[lane], a.num_experts - 1u);
            a.host_readback[2 + K + lane] = t | uint32_t(a.topk_weights[lane]);
            a.host_readback[2 + 2 * K + lane] = t | (lane < hits ? a.hit_positions[lane] : 0u);
            a.host_readback[2 + 3 * K + lane] = t | (lane < misses ? a.miss_positions[lane] : 0u);
            a.host_readback[2 + 4 * K + lane] = t | (a.predicted[lane] & 0xffffu);
        }
    }
}

// ------------------------------------------------------------------ phase 1

struct Phase1Args {
    PoolArg pool;
    uint64_t stride;
    const uint32_t *resolved;
    shrike_expert_offsets off;
    const uint16_t *x;
    uint16_t *acts;
    uint32_t d, f, top_k, meta, act, ebias;
    const uint32_t *indirect, *io_status;
};

// moe.metal:950-999 (4-bit) / :650-672 (8-bit body) with pool addressing :297-305.
// A wave owns RP consecutive f of one routed position: RP gate rows and RP up rows.
template <int BITS, int NCH, int RP>
__global__ __launch_bounds__(256) void k_phase1(Phase1Args a) {
    typedef Chunk<BITS> C;
    __shared__ uint4 xl[SHRIKE_MAX_HIDDEN / 8];
    if (a.indirect && a.indirect[0] == 0u) return;
    if (!io_ready(a.io_status)) return;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t cpr = a.d * BITS / 128u, groups = a.d / kGroup, row_bytes = cpr * 16u;
    const uint32_t pair0 = (blockIdx.x * 4u + wave) * RP;
    const bool in_range = pair0 < a.top_k * a.f;
    const uint32_t k = in_range ? pair0 / a.f : 0u;
    const uint32_t f0 = pair0 - k * a.f;
    const uint32_t cell = in_range ? a.resolved[k] : kSentinel;
    const bool live = cell != kSentinel;  // moe.metal:986
    const uint8_t *base = cell_base(a.pool, live ? cell : 0u, a.stride);

    RowRegs<BITS, NCH> rows[2 * RP];
    if (live) {
#pragma unroll
        for (int r = 0; r < 2 * RP; ++r) {
            const bool up = r >= RP;
            const uint32_t f = f0 + uint32_t(r % RP);
            const uint8_t *w = base + (up ? a.off.up_w_off : a.off.gate_w_off) + size_t(f) * row_bytes;
            const uint16_t *s = reinterpret_cast<const uint16_t *>(base + (up ? a.off.up_s_off : a.off.gate_s_off)) + size_t(f) * groups;
            const uint16_t *b = reinterpret_cast<const uint16_t *>(base + (up ? a.off.up_b_off : a.off.gate_b_off)) + size_t(f) * groups;
            load_row<BITS, NCH>(rows[r], w, s, b, cpr, lane, true);
        }
    }
    for (uint32_t p = threadIdx.x; p < a.d / 8u; p += 256u) xl[p] = reinterpret_cast<const uint4 *>(a.x)[p];
    __syncthreads();
    if (!live) return;

    typename C::X x[NCH];
    float xs[NCH];
    load_slices<BITS, NCH>(xl, cpr, lane, true, x, xs);
    float res[2 * RP];
#pragma unroll
    for (int r = 0; r < 2 * RP; ++r) res[r] = wave_sum(row_partial<BITS, NCH>(rows[r], x, xs, a.meta));
    if (lane == 0) {
#pragma unroll
        for (int p = 0; p < RP; ++p) {
            float g = res[p], u = res[RP + p];
            if (a.ebias) {  // moe.metal:261-269
                g += bf16_to_f32(reinterpret_cast<const uint16_t *>(base + a.off.gate_ab_off)[f0 + p]);
                u += bf16_to_f32(reinterpret_cast<const uint16_t *>(base + a.off.up_ab_off)[f0 + p]);
            }
            a.acts[size_t(k) * a.f + f0 + p] = f32_to_f16(glu_rt(g, u, a.act));
        }
    }
}

// ------------------------------------------------------------------ phase 2

struct Phase2Args {
    PoolArg pool;
    uint64_t stride;
    const uint32_t *resolved, *fallback;
    shrike_expert_offsets off;
    const uint16_t *acts, *routing_w, *residual;
    uint16_t *y, *hidden;
    uint32_t d, f, top_k, meta, ebias;
    const uint32_t *indirect, *io_status;
};

constexpr uint32_t kPhase2Rows = 8;  // output rows per workgroup

// moe.metal:889-893
__device__ __forceinline__ void phase2_finish(uint16_t *y, uint16_t *hidden, uint32_t d, uint16_t value) {
    y[d] = value;
    if (hidden) hidden[d] = f32_to_f16(f16_to_f32(hidden[d]) + f16_to_f32(value));
}

// moe.metal:1008-1057. One wave per routed position (blockDim = 64 * top_k); a
// workgroup owns kPhase2Rows output rows. When a down row is shorter than a wave's
// 1 KiB load, the wave covers 64/cpr rows per load and reduces over lane segments.
template <int BITS, int NCH, int BATCH>
__global__ __launch_bounds__(512) void k_phase2(Phase2Args a) {
    typedef Chunk<BITS> C;
    __shared__ float partial[SHRIKE_MAX_TOP_K][kPhase2Rows];
    if (a.indirect && a.indirect[0] == 0u) return;
    const uint32_t lane = threadIdx.x & 63u, k = threadIdx.x >> 6;
    const uint32_t d0 = blockIdx.x * kPhase2Rows;
    if (!io_ready(a.io_status)) {  // moe.metal:1032-1035
        if (threadIdx.x < kPhase2Rows && d0 + threadIdx.x < a.d)
            phase2_finish(a.y, a.hidden, d0 + threadIdx.x, a.residual ? a.residual[d0 + threadIdx.x] : uint16_t(0));
        return;
    }
    const uint32_t cpr = a.f * BITS / 128u, groups = a.f / kGroup, row_bytes = cpr * 16u;
    const bool packed = cpr < 64u && (64u % cpr) == 0u;
    const uint32_t rpl = packed ? min(64u / cpr, kPhase2Rows) : 1u;  // rows per wave load
    const uint32_t seg = packed ? cpr : 64u;
    const uint32_t sub = packed ? lane / cpr : 0u, col = packed ? lane % cpr : lane;
    const bool lane_on = sub < rpl;

    uint32_t cell = a.resolved[k];
    if (cell == kSentinel && a.fallback) cell = a.fallback[k];  // moe.metal:1037-1038
    const bool live = cell != kSentinel;
    const uint8_t *base = cell_base(a.pool, live ? cell : 0u, a.stride);
    const uint16_t *s_all = reinterpret_cast<const uint16_t *>(base + a.off.down_s_off);
    const uint16_t *b_all = reinterpret_cast<const uint16_t *>(base + a.off.down_b_off);

    if (live) {
        typename C::X x[NCH];
        float xs[NCH];
        load_slices<BITS, NCH>(reinterpret_cast<const uint4 *>(a.acts + size_t(k) * a.f), cpr, col, lane_on, x, xs);
        const float wk = f16_to_f32(a.routing_w[k]);
        const uint32_t n_groups = kPhase2Rows / rpl;
        for (uint32_t g0 = 0; g0 < n_groups; g0 += BATCH) {
            RowRegs<BITS, NCH> rows[BATCH];
            uint32_t row[BATCH];
            bool on[BATCH];
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                row[j] = d0 + (g0 + j) * rpl + sub;
                on[j] = lane_on && (g0 + j) < n_groups && row[j] < a.d;
                const uint32_t rr = on[j] ? row[j] : 0u;
                load_row<BITS, NCH>(rows[j], base + a.off.down_w_off + size_t(rr) * row_bytes,
                                    s_all + size_t(rr) * groups, b_all + size_t(rr) * groups, cpr, col, on[j]);
            }
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                float v = seg_sum(row_partial<BITS, NCH>(rows[j], x, xs, a.meta), seg);
                const bool writer = on[j] && (lane % seg) == seg - 1u;
                if (writer) {
                    if (a.ebias) v += bf16_to_f32(reinterpret_cast<const uint16_t *>(base + a.off.down_ab_off)[row[j]]);
                    partial[k][row[j] - d0] = wk * v;  // moe.metal:1049
                }
            }
        }
    } else if (lane < kPhase2Rows) {
        partial[k][lane] = 0.0f;
    }
    __syncthreads();
    if (threadIdx.x < kPhase2Rows && d0 + threadIdx.x < a.d) {
        const uint32_t d = d0 + threadIdx.x;
        float acc = a.residual ? f16_to_f32(a.residual[d]) : 0.0f;
        for (uint32_t i = 0; i < a.top_k; ++i) acc += partial[i][threadIdx.x];
        phase2_finish(a.y, a.hidden, d, f32_to_f16(acc));
    }
}

// ------------------------------------------------- dense group-affine GEMV

struct GemvArgs {
    // two row sets of one shape over the same input (gate rows then up rows):
    // dequant_int4.metal:206-235; set B unused when rows_b == 0.
    const uint8_t *w_a; const uint16_t *s_a, *b_a; uint16_t *y_a;
    const uint8_t *w_b; const uint16_t *s_b, *b_b; uint16_t *y_b;
    uint32_t rows, rows_b, n, meta;
    // input: x (fp16[n]) or, when gate_in != nullptr, act = half(glu(gate_in, up_in))
    // computed on the fly (dequant_int4.metal:247-287).
    const uint16_t *x, *gate_in, *up_in;
    uint32_t act;
    const uint16_t *scalar_gate;  // dequant_int4.metal:322-329
};

constexpr uint32_t kGemvRowsPerWave = 2;

// dequant_int4.metal:101-199 / dequant_int8.metal:66-107: y[row] = half(W[row,:] . x).
template <int BITS, int NCH>
__global__ __launch_bounds__(256) void k_gemv(GemvArgs a) {
    typedef Chunk<BITS> C;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t cpr = a.n * BITS / 128u, groups = a.n / kGroup, row_bytes = cpr * 16u;
    const bool packed = cpr < 64u && (64u % cpr) == 0u;
    const uint32_t rpl = packed ? 64u / cpr : 1u;
    const uint32_t seg = packed ? cpr : 64u;
    const uint32_t sub = packed ? lane / cpr : 0u, col = packed ? lane % cpr : lane;
    const uint32_t total = a.rows + a.rows_b;
    const uint32_t first = (blockIdx.x * 4u + wave) * kGemvRowsPerWave * rpl;
    if (first >= total) return;

    RowRegs<BITS, NCH> rows[kGemvRowsPerWave];
    uint32_t row[kGemvRowsPerWave];
    bool on[kGemvRowsPerWave];
#pragma unroll
    for (uint32_t j = 0; j < kGemvRowsPerWave; ++j) {
        row[j] = first + j * rpl + sub;
        on[j] = row[j] < total;
        const uint32_t rr = on[j] ? row[j] : 0u;
        const bool second = rr >= a.rows;
        const uint32_t local = second ? rr - a.rows : rr;
        load_row<BITS, NCH>(rows[j], (second ? a.w_b : a.w_a) + size_t(local) * row_bytes,
                            (second ? a.s_b : a.s_a) + size_t(local) * groups,
                            (second ? a.b_b : a.b_a) + size_t(local) * groups, cpr, col, on[j]);
    }
    typename C::X x[NCH];
    float xs[NCH];
    if (a.gate_in) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const uint32_t c = col + 64u * i;
            const bool onc = c < cpr;
            const uint32_t cc = onc ? c : 0u;
            float s = 0.0f;
#pragma unroll
            for (int j = 0; j < C::PIECES; ++j) {
                const uint4 gv = reinterpret_cast<const uint4 *>(a.gate_in)[cc * C::PIECES + j];
                const uint4 uv = reinterpret_cast<const uint4 *>(a.up_in)[cc * C::PIECES + j];
                const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w};
                uint32_t o[4];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const uint16_t lo = f32_to_f16(glu_rt(f16_to_f32(uint16_t(gw[t])), f16_to_f32(uint16_t(uw[t])), a.act));
                    const uint16_t hi = f32_to_f16(glu_rt(f16_to_f32(uint16_t(gw[t] >> 16)), f16_to_f32(uint16_t(uw[t] >> 16)), a.act));
                    o[t] = uint32_t(lo) | (uint32_t(hi) << 16);
                }
                uint4 v = make_uint4(o[0], o[1], o[2], o[3]);
                if (!onc) v = zero4();
                C::fill(x[i], j, v);
                s += sum_x8(v);
            }
            xs[i] = s;
        }
    } else {
        load_slices<BITS, NCH>(reinterpret_cast<const uint4 *>(a.x), cpr, col, true, x, xs);
    }
#pragma unroll
    for (uint32_t j = 0; j < kGemvRowsPerWave; ++j) {
        const float v = seg_sum(row_partial<BITS, NCH>(rows[j], x, xs, a.meta), seg);
        if (on[j] && (lane % seg) == seg - 1u) {
            const bool second = row[j] >= a.rows;
            uint16_t yh = f32_to_f16(v);
            if (a.scalar_gate) yh = f32_to_f16(f16_to_f32(yh) / (1.0f + expf(-f16_to_f32(a.scalar_gate[0]))));
            (second ? a.y_b : a.y_a)[second ? row[j] - a.rows : row[j]] = yh;
        }
    }
}

// --------------------------------------------------------------- launchers

static uint32_t nch_for(uint32_t n, uint32_t bits) { return (n * bits / 128u + 63u) / 64u; }

static void fill_pool(PoolArg &p, const shrike_pool_bases *pool) {
    for (uint32_t i = 0; i < SHRIKE_POOL_MAX_CHUNKS; ++i) p.base[i] = static_cast<const uint8_t *>(pool->base[i]);
    p.cells_per_chunk = pool->cells_per_chunk ? pool->cells_per_chunk : 1u;
}

static int check_offsets(const shrike_expert_offsets *o, uint32_t d, uint32_t f, uint32_t bits) {
    SHRIKE_REQUIRE(o != nullptr, "offsets is NULL");
    SHRIKE_REQUIRE(d % SHRIKE_GROUP_SIZE == 0 && f % SHRIKE_GROUP_SIZE == 0,
                   "d=%u and f=%u must be multiples of %u", d, f, SHRIKE_GROUP_SIZE);
    SHRIKE_REQUIRE(d <= SHRIKE_MAX_HIDDEN, "d=%u exceeds the staged activation ceiling %u", d, SHRIKE_MAX_HIDDEN);
    SHRIKE_REQUIRE(nch_for(d, bits) <= 4 && nch_for(f, bits) <= 4, "row of %u/%u %u-bit codes is too long", d, f, bits);
    // 128-bit code loads need 16-byte aligned code tensors; metadata needs 2 bytes
    SHRIKE_REQUIRE((o->gate_w_off | o->up_w_off | o->down_w_off) % 16u == 0,
                   "code sub-tensors must be 16-byte aligned inside the blob");
    SHRIKE_REQUIRE((o->gate_s_off | o->gate_b_off | o->up_s_off | o->up_b_off | o->down_s_off | o->down_b_off
                    | o->gate_ab_off | o->up_ab_off | o->down_ab_off) % 2u == 0,
                   "metadata sub-tensors must be 2-byte aligned");
    SHRIKE_REQUIRE((d * bits / 8u) % 16u == 0 && (f * bits / 8u) % 16u == 0, "row bytes must be a multiple of 16");
    return 0;
}

template <int BITS>
static int launch_phase1(const Phase1Args &a, hipStream_t s) {
    constexpr int RP = 2;
    const uint32_t waves = (a.top_k * a.f + RP - 1) / RP;
    const dim3 grid((waves + 3) / 4), block(256);
    switch (nch_for(a.d, BITS)) {
        case 1: hipLaunchKernelGGL((k_phase1<BITS, 1, RP>), grid, block, 0, s, a); break;
        case 2: hipLaunchKernelGGL((k_phase1<BITS, 2, RP>), grid, block, 0, s, a); break;
        case 3: hipLaunchKernelGGL((k_phase1<BITS, 3, RP>), grid, block, 0, s, a); break;
        default: hipLaunchKernelGGL((k_phase1<BITS, 4, RP>), grid, block, 0, s, a); break;
    }
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

template <int BITS, int NCH>
static void launch_phase2_batch(const Phase2Args &a, dim3 grid, dim3 block, hipStream_t s) {
    const uint32_t cpr = a.f * BITS / 128u;
    const uint32_t rpl = (cpr < 64u && 64u % cpr == 0u) ? (64u / cpr < kPhase2Rows ? 64u / cpr : kPhase2Rows) : 1u;
    const uint32_t n_groups = kPhase2Rows / rpl;  // row groups per wave; up to 4 in flight
    if (n_groups >= 4) hipLaunchKernelGGL((k_phase2<BITS, NCH, 4>), grid, block, 0, s, a);
    else if (n_groups == 2) hipLaunchKernelGGL((k_phase2<BITS, NCH, 2>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((k_phase2<BITS, NCH, 1>), grid, block, 0, s, a);
}

template <int BITS>
static int launch_phase2(const Phase2Args &a, hipStream_t s) {
    const dim3 grid((a.d + kPhase2Rows - 1) / kPhase2Rows), block(64 * a.top_k);
    switch (nch_for(a.f, BITS)) {
        case 1: launch_phase2_batch<BITS, 1>(a, grid, block, s); break;
        case 2: launch_phase2_batch<BITS, 2>(a, grid, block, s); break;
        case 3: launch_phase2_batch<BITS, 3>(a, grid, block, s); break;
        default: launch_phase2_batch<BITS, 4>(a, grid, block, s); break;
    }
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

template <int BITS>
static int launch_gemv(const GemvArgs &a, hipStream_t s) {
    const uint32_t cpr = a.n * BITS / 128u;
    const uint32_t rpl = (cpr < 64u && 64u % cpr == 0u) ? 64u / cpr : 1u;
    const uint32_t per_wave = kGemvRowsPerWave * rpl;
    const uint32_t waves = (a.rows + a.rows_b + per_wave - 1) / per_wave;
    const dim3 grid((waves + 3) / 4), block(256);
    switch (nch_for(a.n, BITS)) {
        case 1: hipLaunchKernelGGL((k_gemv<BITS, 1>), grid, block, 0, s, a); break;
        case 2: hipLaunchKernelGGL((k_gemv<BITS, 2>), grid, block, 0, s, a); break;
        case 3: hipLaunchKernelGGL((k_gemv<BITS, 3>), grid, block, 0, s, a); break;
        default: hipLaunchKernelGGL((k_gemv<BITS, 4>), grid, block, 0, s, a); break;
    }
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

static int launch_router(const RouterArgs &a, uint32_t router_bits, hipStream_t s) {
    const dim3 grid((a.num_experts + 3) / 4), block(256);
    if (router_bits == 0) hipLaunchKernelGGL((k_router<0>), grid, block, 0, s, a);
    else if (router_bits == 8) hipLaunchKernelGGL((k_router<8>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((k_router<4>), grid, block, 0, s, a);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

static int check_router(const shrike_hip_moe *moe, uint32_t num_experts, uint32_t d, uint32_t top_k) {
    // MoE.swift:262-277
    SHRIKE_REQUIRE(d % SHRIKE_GROUP_SIZE == 0, "encodeRouter: d=%u must be a multiple of %u", d, SHRIKE_GROUP_SIZE);
    SHRIKE_REQUIRE(num_experts >= 1 && num_experts <= SHRIKE_MAX_ROUTER_EXPERTS, "encodeRouter: numExperts=%u not in 1...256", num_experts);
    SHRIKE_REQUIRE(top_k >= 1 && top_k <= SHRIKE_MAX_TOP_K, "encodeRouter: topK=%u not in 1...8", top_k);
    SHRIKE_REQUIRE(top_k <= num_experts, "encodeRouter: topK=%u exceeds numExperts=%u", top_k, num_experts);
    const uint32_t bits = moe->desc.router_weight_bits;
    const uint32_t chunks = bits == 0 ? d / 8u : d * bits / 128u;
    SHRIKE_REQUIRE(chunks <= (bits == 0 ? 512u : 256u), "encodeRouter: d=%u is too long for the router kernel", d);
    return 0;
}

}  // namespace shrike

using namespace shrike;

extern "C" {

int shrike_hip_moe_router(shrike_hip_moe *moe, void *stream, const void *d_weights, const void *d_scales,
                          const void *d_biases, const void *d_hidden, const void *d_effective_scale,
                          const void *d_per_expert_scale, const void *d_logit_bias, uint32_t *d_out_indices,
                          void *d_out_weights, uint32_t num_experts, uint32_t d, uint32_t top_k) {
    SHRIKE_REQUIRE(moe != nullptr, "moe handle is NULL");
    if (int rc = check_router(moe, num_experts, d, top_k)) return rc;
    SHRIKE_REQUIRE(d_weights && d_hidden && d_effective_scale && d_per_expert_scale && d_logit_bias,
                   "encodeRouter: weights, hidden, effectiveScale, perExpertScale and logitBias must all be bound");
    SHRIKE_REQUIRE(moe->desc.router_weight_bits == 0 || (d_scales && d_biases), "encodeRouter: affine router needs scales and biases");
    SHRIKE_REQUIRE(d_out_indices && d_out_weights, "encodeRouter: outputs must be bound");
    RouterArgs a = {};
    a.weights = d_weights;
    a.scales = static_cast<const uint16_t *>(d_scales);
    a.biases = static_cast<const uint16_t *>(d_biases);
    a.hidden = static_cast<const uint16_t *>(d_hidden);
    a.effective_scale = static_cast<const uint16_t *>(d_effective_scale);
    a.per_expert_scale = static_cast<const uint16_t *>(d_per_expert_scale);
    a.logit_bias = static_cast<const uint16_t *>(d_logit_bias);
    a.logits = moe->d_logits;
    a.counter = moe->d_counter;
    a.out_indices = d_out_indices;
    a.out_weights = static_cast<uint16_t *>(d_out_weights);
    a.num_experts = num_experts; a.d = d; a.top_k = top_k;
    a.meta = moe->desc.meta_dtype; a.sigmoid = moe->desc.sigmoid_router_scores;
    a.scaling = moe->desc.routed_scaling_factor;
    return launch_router(a, moe->desc.router_weight_bits, as_stream(stream));
}

const float *shrike_hip_moe_router_logits(const shrike_hip_moe *moe) { return moe ? moe->d_logits : nullptr; }

int shrike_hip_moe_classify(shrike_hip_moe *moe, void *stream, const uint32_t *d_topk_indices,
                            const uint64_t *d_residency, uint32_t *d_hit_count, uint32_t *d_hit_positions,
                            uint32_t *d_miss_count, uint32_t *d_miss_positions, uint32_t *d_miss_experts,
                            uint32_t *d_resolved_slots, uint32_t top_k, uint32_t num_experts,
                            const uint32_t full_grids[12], uint32_t *d_spec_args, uint32_t *d_host_readback,
                            uint32_t host_readback_tag, const void *d_topk_weights,
                            const uint32_t *d_predicted_indices) {
    SHRIKE_REQUIRE(moe != nullptr, "moe handle is NULL");
    SHRIKE_REQUIRE(top_k >= 1 && top_k <= SHRIKE_MAX_TOP_K, "classify: topK=%u not in 1...8", top_k);  // MoE.swift:567
    SHRIKE_REQUIRE(num_experts >= 1, "classify: numExperts must be positive");
    SHRIKE_REQUIRE(d_topk_indices && d_residency && d_hit_count && d_hit_positions && d_miss_count
                   && d_miss_positions && d_miss_experts && d_resolved_slots, "classify: every list must be bound");
    SHRIKE_REQUIRE(host_readback_tag == 0 || (d_host_readback && d_topk_weights && d_predicted_indices),
                   "classify: a tagged readback needs its buffer, the weights and the predicted ids");  // MoE.swift:569-575
    SHRIKE_REQUIRE(host_readback_tag <= 0xffffu, "classify: the readback tag is 16 bits");
    ClassifyArgs a = {};
    a.topk = d_topk_indices; a.residency = d_residency;
    a.hit_count = d_hit_count; a.hit_positions = d_hit_positions; a.miss_count = d_miss_count;
    a.miss_positions = d_miss_positions; a.miss_experts = d_miss_experts; a.resolved_slots = d_resolved_slots;
    a.top_k = top_k; a.num_experts = num_experts;
    for (int i = 0; i < 12; ++i) a.full_grids[i] = full_grids ? full_grids[i] : 1u;
    a.spec_args = d_spec_args; a.host_readback = d_host_readback; a.tag = host_readback_tag;
    a.topk_weights = static_cast<const uint16_t *>(d_topk_weights); a.predicted = d_predicted_indices;
    hipLaunchKernelGGL(k_classify, dim3(1), dim3(64), 0, as_stream(stream), a);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

int shrike_hip_moe_phase1_pool(shrike_hip_moe *moe, void *stream, const shrike_pool_bases *pool,
                               uint64_t pool_slot_stride, const uint32_t *d_resolved_slots,
                               const shrike_expert_offsets *offsets, const void *d_x, void *d_acts, uint32_t d,
                               uint32_t f, uint32_t top_k, const uint32_t *d_indirect, const uint32_t *d_io_status) {
    SHRIKE_REQUIRE(moe != nullptr && pool != nullptr, "moe handle or pool is NULL");
    SHRIKE_REQUIRE(top_k >= 1 && top_k <= SHRIKE_MAX_TOP_K, "phase1: topK=%u not in 1...8", top_k);  // MoE.swift:925
    const uint32_t bits = moe->desc.routed_weight_bits;
    if (int rc = check_offsets(offsets, d, f, bits)) return rc;
    SHRIKE_REQUIRE(d_resolved_slots && d_x && d_acts, "phase1: resolvedSlots, x and acts must be bound");
    SHRIKE_REQUIRE(pool_slot_stride % 16u == 0, "phase1: pool slot stride must be a multiple of 16");
    Phase1Args a = {};
    fill_pool(a.pool, pool);
    a.stride = pool_slot_stride; a.resolved = d_resolved_slots; a.off = *offsets;
    a.x = static_cast<const uint16_t *>(d_x); a.acts = static_cast<uint16_t *>(d_acts);
    a.d = d; a.f = f; a.top_k = top_k; a.meta = moe->desc.meta_dtype; a.act = moe->desc.activation;
    a.ebias = moe->desc.expert_additive_biases;
    a.indirect = d_indirect; a.io_status = moe->desc.event_gated_io ? d_io_status : nullptr;
    return bits == 4 ? launch_phase1<4>(a, as_stream(stream)) : launch_phase1<8>(a, as_stream(stream));
}

int shrike_hip_moe_phase2_pool(shrike_hip_moe *moe, void *stream, const shrike_pool_bases *pool,
                               uint64_t pool_slot_stride, const uint32_t *d_resolved_slots,
                               const uint32_t *d_fallback_cells, const shrike_expert_offsets *offsets,
                               const void *d_acts, const void *d_routing_weights, const void *d_residual, void *d_y,
                               void *d_hidden, uint32_t d, uint32_t f, uint32_t top_k, const uint32_t *d_indirect,
                               const uint32_t *d_io_status) {
    SHRIKE_REQUIRE(moe != nullptr && pool != nullptr, "moe handle or pool is NULL");
    SHRIKE_REQUIRE(top_k >= 1 && top_k <= SHRIKE_MAX_TOP_K, "phase2: topK=%u not in 1...8", top_k);  // MoE.swift:1015
    const uint32_t bits = moe->desc.routed_weight_bits;
    if (int rc = check_offsets(offsets, d, f, bits)) return rc;
    SHRIKE_REQUIRE(d_resolved_slots && d_acts && d_routing_weights && d_residual && d_y,
                   "phase2: resolvedSlots, acts, routingWeights, residual and y must be bound");
    SHRIKE_REQUIRE(pool_slot_stride % 16u == 0, "phase2: pool slot stride must be a multiple of 16");
    Phase2Args a = {};
    fill_pool(a.pool, pool);
    a.stride = pool_slot_stride; a.resolved = d_resolved_slots; a.fallback = d_fallback_cells; a.off = *offsets;
    a.acts = static_cast<const uint16_t *>(d_acts); a.routing_w = static_cast<const uint16_t *>(d_routing_weights);
    a.residual = static_cast<const uint16_t *>(d_residual);
    a.y = static_cast<uint16_t *>(d_y); a.hidden = static_cast<uint16_t *>(d_hidden);
    a.d = d; a.f = f; a.top_k = top_k; a.meta = moe->desc.meta_dtype; a.ebias = moe->desc.expert_additive_biases;
    a.indirect = d_indirect; a.io_status = moe->desc.event_gated_io ? d_io_status : nullptr;
    return bits == 4 ? launch_phase2<4>(a, as_stream(stream)) : launch_phase2<8>(a, as_stream(stream));
}

int shrike_hip_shared_expert(shrike_hip_moe *moe, void *stream, const shrike_projection *gate,
                             const shrike_projection *up, const shrike_projection *down, uint32_t bits,
                             const void *d_x, void *d_scratch, void *d_h1, const void *d_scalar_gate, uint32_t d,
                             uint32_t f_shared) {
    SHRIKE_REQUIRE(moe != nullptr, "moe handle is NULL");
    SHRIKE_REQUIRE(gate && up && down && gate->weights && up->weights && down->weights,
                   "sharedExpert: gate, up and down projections must be bound");
    SHRIKE_REQUIRE(bits == 4 || bits == 8, "sharedExpert: bits=%u not in {4, 8}", bits);
    SHRIKE_REQUIRE(d % SHRIKE_GROUP_SIZE == 0 && f_shared % SHRIKE_GROUP_SIZE == 0,
                   "sharedExpert: d=%u and f=%u must be multiples of %u", d, f_shared, SHRIKE_GROUP_SIZE);
    SHRIKE_REQUIRE(nch_for(d, bits) <= 4 && nch_for(f_shared, bits) <= 4, "sharedExpert: rows too long");
    SHRIKE_REQUIRE(d_x && d_scratch && d_h1, "sharedExpert: x, scratch and h1 must be bound");
    uint16_t *gate_out = static_cast<uint16_t *>(d_scratch), *up_out = gate_out + f_shared;
    GemvArgs a = {};
    a.w_a = static_cast<const uint8_t *>(gate->weights); a.s_a = static_cast<const uint16_t *>(gate->scales);
    a.b_a = static_cast<const uint16_t *>(gate->biases); a.y_a = gate_out;
    a.w_b = static_cast<const uint8_t *>(up->weights); a.s_b = static_cast<const uint16_t *>(up->scales);
    a.b_b = static_cast<const uint16_t *>(up->biases); a.y_b = up_out;
    a.rows = f_shared; a.rows_b = f_shared; a.n = d; a.meta = moe->desc.meta_dtype;
    a.x = static_cast<const uint16_t *>(d_x);
    if (int rc = bits == 4 ? launch_gemv<4>(a, as_stream(stream)) : launch_gemv<8>(a, as_stream(stream))) return rc;
    GemvArgs b = {};
    b.w_a = static_cast<const uint8_t *>(down->weights); b.s_a = static_cast<const uint16_t *>(down->scales);
    b.b_a = static_cast<const uint16_t *>(down->biases); b.y_a = static_cast<uint16_t *>(d_h1);
    b.rows = d; b.rows_b = 0; b.n = f_shared; b.meta = moe->desc.meta_dtype;
    b.gate_in = gate_out; b.up_in = up_out; b.act = moe->desc.activation;
    b.scalar_gate = static_cast<const uint16_t *>(d_scalar_gate);
    return bits == 4 ? launch_gemv<4>(b, as_stream(stream)) : launch_gemv<8>(b, as_stream(stream));
}

int shrike_hip_moe_decode_layer(shrike_hip_moe *moe, void *stream, const shrike_decode_layer_args *g) {
    SHRIKE_REQUIRE(moe != nullptr && g != nullptr, "moe handle or args is NULL");
    const shrike_moe_desc &m = moe->desc;
    if (int rc = check_router(moe, m.num_experts, m.d, m.top_k)) return rc;
    if (int rc = check_offsets(&g->offsets, m.d, m.f, m.routed_weight_bits)) return rc;
    SHRIKE_REQUIRE(g->router_weights && g->effective_scale && g->per_expert_scale && g->logit_bias,
                   "decodeLayer: router operands must be bound");
    SHRIKE_REQUIRE(g->pool && g->residency && g->x && g->y && g->out_indices && g->out_weights && g->resolved_slots
                   && g->hit_count && g->hit_positions && g->miss_count && g->miss_positions && g->miss_experts
                   && g->acts, "decodeLayer: pool, residency, x, y and the scratch buffers must be bound");
    hipStream_t s = as_stream(stream);
    // 1. router + select + classify: one launch
    RouterArgs r = {};
    r.weights = g->router_weights; r.scales = static_cast<const uint16_t *>(g->router_scales);
    r.biases = static_cast<const uint16_t *>(g->router_biases);
    r.hidden = static_cast<const uint16_t *>(g->x);
    r.effective_scale = static_cast<const uint16_t *>(g->effective_scale);
    r.per_expert_scale = static_cast<const uint16_t *>(g->per_expert_scale);
    r.logit_bias = static_cast<const uint16_t *>(g->logit_bias);
    r.logits = moe->d_logits; r.counter = moe->d_counter;
    r.out_indices = g->out_indices; r.out_weights = static_cast<uint16_t *>(g->out_weights);
    r.num_experts = m.num_experts; r.d = m.d; r.top_k = m.top_k; r.meta = m.meta_dtype;
    r.sigmoid = m.sigmoid_router_scores; r.scaling = m.routed_scaling_factor;
    r.residency = g->residency; r.hit_count = g->hit_count; r.hit_positions = g->hit_positions;
    r.miss_count = g->miss_count; r.miss_positions = g->miss_positions; r.miss_experts = g->miss_experts;
    r.resolved_slots = g->resolved_slots;
    if (int rc = launch_router(r, m.router_weight_bits, s)) return rc;
    // 2. shared expert -> h1 (the residual of phase 2); without one the residual is zero
    const void *residual = nullptr;
    if (g->shared_gate.weights) {
        SHRIKE_REQUIRE(g->shared_scratch, "decodeLayer: sharedScratch must be bound");
        if (int rc = shrike_hip_shared_expert(moe, stream, &g->shared_gate, &g->shared_up, &g->shared_down,
                                              g->shared_bits ? g->shared_bits : m.routed_weight_bits, g->x,
                                              g->shared_scratch, g->h1, g->shared_scalar_gate, m.d, g->shared_f))
            return rc;
        residual = g->h1;
    }
    // 3. phase 1, 4. phase 2
    if (int rc = shrike_hip_moe_phase1_pool(moe, stream, g->pool, g->pool_slot_stride, g->resolved_slots, &g->offsets,
                                            g->x, g->acts, m.d, m.f, m.top_k, nullptr, nullptr))
        return rc;
    Phase2Args p = {};
    fill_pool(p.pool, g->pool);
    p.stride = g->pool_slot_stride; p.resolved = g->resolved_slots; p.off = g->offsets;
    p.acts = static_cast<const uint16_t *>(g->acts); p.routing_w = static_cast<const uint16_t *>(g->out_weights);
    p.residual = static_cast<const uint16_t *>(residual);
    p.y = static_cast<uint16_t *>(g->y); p.hidden = static_cast<uint16_t *>(g->hidden);
    p.d = m.d; p.f = m.f; p.top_k = m.top_k; p.meta = m.meta_dtype; p.ebias = m.expert_additive_biases;
    return m.routed_weight_bits == 4 ? launch_phase2<4>(p, s) : launch_phase2<8>(p, s);
}

}  // extern "C"
