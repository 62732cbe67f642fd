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

struct SelectArgs {
    const float *logits;
    const uint16_t *per_expert_scale, *logit_bias;
    uint32_t num_experts, top_k, sigmoid;
    float scaling;
};

struct RouteLists {  // outputs of select + classify; residency == nullptr: select only
    uint32_t *out_indices;
    uint16_t *out_weights;
    const uint64_t *residency;
    uint32_t *hit_count, *hit_positions, *miss_count, *miss_positions, *miss_experts, *resolved_slots;
};

struct RouterArgs {
    const void *weights;
    const uint16_t *scales, *biases;
    const uint16_t *hidden, *effective_scale;
    uint32_t d, meta;
    uint32_t *counter;
    float *logits_out;
    SelectArgs sel;
    RouteLists lists;
};

__device__ __forceinline__ uint32_t orderable(float v) {
    const uint32_t u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float from_orderable(uint32_t o) {
    return __uint_as_float((o & 0x80000000u) ? (o & 0x7fffffffu) : ~o);
}
__device__ __forceinline__ float sigmoidf_(float v) { return 1.0f / (1.0f + expf(-v)); }
template <bool COHERENT>
__device__ __forceinline__ float load_logit(const float *p) {
    return COHERENT ? __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : *p;
}

// moe.metal:419-491 and :121-151, run by one wave. Lane l holds experts l, l+64, l+128,
// l+192 with their bias, scale and residency word (all fetched up front, so nothing
// that follows waits on memory); top_k rounds of a wave-wide max over the key (orderable
// score, then lower index) pick the experts in rank order. On return lane p < top_k holds
// position p's expert, fp16 weight and resolved cell (sentinel on a miss). COHERENT reads
// the logits past the non-coherent caches (they were written by other workgroups of the
// same launch); otherwise they come from an earlier launch.
template <bool COHERENT>
__device__ void route_wave(const SelectArgs &a, const RouteLists &out, uint32_t lane, bool write_lists,
                           uint32_t &my_cell) {
    uint64_t key[4], word[4];
    float raw[4], gain[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t e = lane + 64u * j;
        const bool on = e < a.num_experts;
        const uint32_t ee = on ? e : 0u;
        raw[j] = load_logit<COHERENT>(a.logits + ee);
        const float bias = bf16_to_f32(a.logit_bias[ee]);
        gain[j] = bf16_to_f32(a.per_expert_scale[ee]);
        word[j] = out.residency ? out.residency[ee] : 0;
        float s = (a.sigmoid ? sigmoidf_(raw[j]) : raw[j]) + bias;
        s = s + 0.0f;  // -0 and +0 tie
        key[j] = (on && s == s) ? (uint64_t(orderable(s)) << 32) | uint64_t(0xffffffffu - e) : 0;
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
    // position p = lane: its expert, then that expert's raw logit, gain and residency word
    // from the lane that holds them
    uint32_t mine = 0;
    float my_score = -INFINITY;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        mine = lane == uint32_t(r) ? idx[r] : mine;
        my_score = lane == uint32_t(r) ? score[r] : my_score;
    }
    const uint32_t src = mine & 63u, jj = mine >> 6;
    float my_raw = 0.0f, my_gain = 0.0f;
    uint32_t w_lo = 0, w_hi = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float r_ = __shfl(raw[j], src), g_ = __shfl(gain[j], src);
        const uint32_t lo_ = __shfl(uint32_t(word[j]), src), hi_ = __shfl(uint32_t(word[j] >> 32), src);
        if (jj == uint32_t(j)) { my_raw = r_; my_gain = g_; w_lo = lo_; w_hi = hi_; }
    }
    const bool on = lane < K;
    float weight;
    if (a.sigmoid) {  // moe.metal:460-474
        const float orig = on ? sigmoidf_(my_raw) : 0.0f;
        float sum = 0.0f;
#pragma unroll
        for (int r = 0; r < 8; ++r) {  // rank order, as the reference adds them
            const float o = __shfl(orig, r);
            if (uint32_t(r) < K) sum += o;
        }
        weight = orig * (a.scaling / (sum + 1e-20f));
    } else {  // moe.metal:477-490
        const float top = __shfl(my_score, 0);
        const float ex = on ? expf(my_score - top) : 0.0f;
        float sum = 0.0f;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const float o = __shfl(ex, r);
            if (uint32_t(r) < K) sum += o;
        }
        weight = ex / sum;
    }
    const uint16_t wbits = f32_to_f16(weight * my_gain);
    if (write_lists && on) {
        out.out_indices[lane] = mine;
        out.out_weights[lane] = wbits;
    }
    my_cell = kSentinel;
    if (!out.residency) return;
    // moe.metal:121-151 (the select above never yields an index past num_experts - 1, so
    // the reference's clamp is the identity here)
    const bool hit = on && w_hi == SHRIKE_RESIDENCY_RESIDENT && w_lo != kSentinel;
    if (hit) my_cell = w_lo;
    if (!write_lists) return;
    const uint64_t hit_mask = __ballot(hit), miss_mask = __ballot(on && !hit);
    const uint64_t below = (uint64_t(1) << lane) - 1u;
    if (hit) {
        out.hit_positions[__popcll(hit_mask & below)] = lane;
        out.resolved_slots[lane] = w_lo;
    } else if (on) {
        const uint32_t at = __popcll(miss_mask & below);
        out.miss_positions[at] = lane;
        out.miss_experts[at] = mine;
        out.resolved_slots[lane] = kSentinel;
    }
    if (lane == 0) {
        out.hit_count[0] = __popcll(hit_mask);
        out.miss_count[0] = __popcll(miss_mask);
    }
}

// One expert row of the router GEMV (moe.metal:324-364), RK: 0 = fp16 rows, 8 / 4 =
// group-affine codes. The per-lane fused-multiply-add order and the xor butterfly are
// fixed so that the fp32 logits are reproducible bit for bit (lane l takes chunks
// l, l+64, ...).
template <int RK>
__device__ __forceinline__ void router_row(const RouterArgs &a, uint32_t e, uint32_t lane) {
    constexpr int E = RK == 0 ? 8 : RK == 8 ? 16 : 32;  // elements per 16-byte weight chunk
    constexpr int PIECES = E / 8;
    constexpr int MAXI = RK == 0 ? 8 : 4;
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
    if (lane == 0) a.logits_out[e] = acc;
}

// MoE.encodeRouter as one launch: four expert rows per workgroup, and the workgroup that
// finishes last runs select (+ classify when a residency table is bound).
template <int RK>
__global__ __launch_bounds__(256) void k_router(RouterArgs a) {
    __shared__ uint32_t s_last;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t e = blockIdx.x * 4u + wave;
    if (e < a.sel.num_experts) {
        router_row<RK>(a, e, lane);
        if (lane == 0) __threadfence();
    }
    if (!a.lists.out_indices) return;  // scores only
    __syncthreads();
    if (threadIdx.x == 0) {
        __threadfence();
        s_last = atomicAdd(a.counter, 1u) == gridDim.x - 1u ? 1u : 0u;
    }
    __syncthreads();
    if (!s_last || wave != 0) return;
    __threadfence();
    uint32_t cell;
    route_wave<true>(a.sel, a.lists, lane, true, cell);
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

// moe.metal:194-231 with the readback of :158-181; lane p classifies position p.
__global__ __launch_bounds__(64) void k_classify(ClassifyArgs a) {
    const uint32_t lane = threadIdx.x;
    const bool on = lane < a.top_k;
    uint32_t expert = 0, slot = kSentinel, state = 0;
    if (on) {
        expert = min(a.topk[lane], a.num_experts - 1u);
        const uint64_t word = a.residency[expert];
        slot = uint32_t(word);
        state = uint32_t(word >> 32);
    }
    const bool hit = on && state == SHRIKE_RESIDENCY_RESIDENT && slot != kSentinel;
    const uint64_t hit_mask = __ballot(hit), miss_mask = __ballot(on && !hit);
    const uint64_t below = (uint64_t(1) << lane) - 1u;
    const uint32_t hits = __popcll(hit_mask), misses = __popcll(miss_mask);
    const uint32_t my_hit_at = __popcll(hit_mask & below), my_miss_at = __popcll(miss_mask & below);
    if (hit) {
        a.hit_positions[my_hit_at] = lane;
        a.resolved_slots[lane] = slot;
    } else if (on) {
        a.miss_positions[my_miss_at] = lane;
        a.miss_experts[my_miss_at] = expert;
        a.resolved_slots[lane] = kSentinel;
    }
    if (lane == 0) {
        a.hit_count[0] = hits;
        a.miss_count[0] = misses;
    }
    const bool all_hit = misses == 0u;
    if (a.spec_args && lane < 3) {
        const uint32_t zero_grid = lane == 0 ? 0u : 1u;
        a.spec_args[lane] = a.full_grids[lane];
        a.spec_args[3 + lane] = all_hit ? a.full_grids[3 + lane] : zero_grid;
        a.spec_args[6 + lane] = all_hit ? zero_grid : a.full_grids[6 + lane];
        a.spec_args[9 + lane] = all_hit ? zero_grid : a.full_grids[9 + lane];
    }
    if (a.tag != 0u && a.host_readback) {
        // the i-th hit / miss position lives in the lane whose rank in the mask is i
        __shared__ uint32_t s_hit[SHRIKE_MAX_TOP_K], s_miss[SHRIKE_MAX_TOP_K];
        if (hit) s_hit[my_hit_at] = lane;
        else if (on) s_miss[my_miss_at] = lane;
        __syncthreads();
        const uint32_t t = a.tag << 16, K = a.top_k;
        if (lane == 0) {
            a.host_readback[0] = t | hits;
            a.host_readback[1] = t | misses;
        }
        if (on) {
            a.host_readback[2 + lane] = t | expert;
            a.host_readback[2 + K + lane] = t | uint32_t(a.topk_weights[lane]);
            a.host_readback[2 + 2 * K + lane] = t | (lane < hits ? s_hit[lane] : 0u);
            a.host_readback[2 + 3 * K + lane] = t | (lane < misses ? s_miss[lane] : 0u);
            a.host_readback[2 + 4 * K + lane] = t | (a.predicted[lane] & 0xffffu);
        }
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

constexpr uint32_t kGemvRowsPerWave = 4;

// dequant_int4.metal:101-199 / dequant_int8.metal:66-107: y[row] = half(W[row,:] . x), the
// work of workgroup `block` of a grid of 256-thread workgroups.
template <int BITS, int NCH>
__device__ __forceinline__ void gemv_job(const GemvArgs &a, uint32_t block) {
    typedef Chunk<BITS> C;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t cpr = a.n * BITS / 128u, groups = a.n / kGroup, row_bytes = cpr * 16u;
    const bool packed = cpr < 64u && (64u % cpr) == 0u;
    const uint32_t rpl = packed ? 64u / cpr : 1u;
    const uint32_t seg = packed ? cpr : 64u;
    const uint32_t sub = packed ? lane / cpr : 0u, col = packed ? lane % cpr : lane;
    const uint32_t total = a.rows + a.rows_b;
    const uint32_t first = (block * 4u + wave) * kGemvRowsPerWave * rpl;
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

static uint32_t gemv_blocks(uint32_t total_rows, uint32_t n, uint32_t bits) {
    const uint32_t cpr = n * bits / 128u;
    const uint32_t rpl = (cpr < 64u && 64u % cpr == 0u) ? 64u / cpr : 1u;
    const uint32_t per_wave = kGemvRowsPerWave * rpl;
    return ((total_rows + per_wave - 1) / per_wave + 3) / 4;
}

template <int BITS, int NCH>
__global__ __launch_bounds__(256) void k_gemv(GemvArgs a) { gemv_job<BITS, NCH>(a, blockIdx.x); }

// The head of the fused layer: the router's logit rows and, beside them in the same grid,
// the shared expert's gate and up rows. Neither depends on the other.
template <int RK, int BITS, int NCH>
__global__ __launch_bounds__(256) void k_head(RouterArgs r, GemvArgs g, uint32_t router_blocks) {
    if (blockIdx.x < router_blocks) {
        const uint32_t e = blockIdx.x * 4u + (threadIdx.x >> 6);
        if (e < r.sel.num_experts) router_row<RK>(r, e, threadIdx.x & 63u);
    } else {
        gemv_job<BITS, NCH>(g, blockIdx.x - router_blocks);
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
    // fused layer only: route from the logits of the previous launch (sel.logits != nullptr),
    // and run the shared expert's down projection in workgroups past `routed_blocks`
    SelectArgs sel;
    RouteLists lists;
    uint32_t routed_blocks;
    GemvArgs shared_down;
};

// moe.metal:950-999 (4-bit) / :650-672 (8-bit body) with pool addressing :297-305.
// A wave owns RP consecutive f of one routed position: RP gate rows and RP up rows.
// SBITS != 0 adds the shared expert's fused down GEMV (one chunk column per lane).
template <int BITS, int NCH, int RP, int SBITS>
__global__ __launch_bounds__(256) void k_phase1(Phase1Args a) {
    typedef Chunk<BITS> C;
    __shared__ uint4 xl[SHRIKE_MAX_HIDDEN / 8];
    __shared__ uint32_t s_cell[SHRIKE_MAX_TOP_K];
    if (SBITS != 0 && blockIdx.x >= a.routed_blocks) {
        gemv_job<SBITS == 0 ? 4 : SBITS, 1>(a.shared_down, blockIdx.x - a.routed_blocks);
        return;
    }
    if (a.indirect && a.indirect[0] == 0u) return;
    if (!io_ready(a.io_status)) return;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t cpr = a.d * BITS / 128u, groups = a.d / kGroup, row_bytes = cpr * 16u;
    const uint32_t pair0 = (blockIdx.x * 4u + wave) * RP;
    const bool in_range = pair0 < a.top_k * a.f;
    const uint32_t k = in_range ? pair0 / a.f : 0u;
    const uint32_t f0 = pair0 - k * a.f;
    const bool routing = a.sel.logits != nullptr;
    uint32_t cell = kSentinel;
    if (!routing && in_range) cell = a.resolved[k];

    for (uint32_t p = threadIdx.x; p < a.d / 8u; p += 256u) xl[p] = reinterpret_cast<const uint4 *>(a.x)[p];
    if (routing && wave == 0) {
        uint32_t my_cell;
        route_wave<false>(a.sel, a.lists, lane, blockIdx.x == 0, my_cell);
        if (lane < a.top_k) s_cell[lane] = my_cell;
    }
    RowRegs<BITS, NCH> rows[2 * RP];
    auto issue_rows = [&](const uint8_t *base) {
#pragma unroll
        for (int r = 0; r < 2 * RP; ++r) {
            const bool up = r >= RP;
            const uint32_t f = f0 + uint32_t(r % RP);
            const uint8_t *w = base + (up ? a.off.up_w_off : a.off.gate_w_off) + size_t(f) * row_bytes;
            const uint16_t *s = reinterpret_cast<const uint16_t *>(base + (up ? a.off.up_s_off : a.off.gate_s_off)) + size_t(f) * groups;
            const uint16_t *b = reinterpret_cast<const uint16_t *>(base + (up ? a.off.up_b_off : a.off.gate_b_off)) + size_t(f) * groups;
            load_row<BITS, NCH>(rows[r], w, s, b, cpr, lane, true);
        }
    };
    if (!routing && cell != kSentinel) issue_rows(cell_base(a.pool, cell, a.stride));
    __syncthreads();
    if (routing) {
        if (in_range) cell = s_cell[k];
        if (cell != kSentinel) issue_rows(cell_base(a.pool, cell, a.stride));
    }
    if (cell == kSentinel) return;  // moe.metal:986 (and waves past the last row)
    const uint8_t *base = cell_base(a.pool, cell, a.stride);

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
__device__ __forceinline__ void phase2_finish(uint16_t *y, uint16_t *hidden, uint32_t d, uint16_t value,
                                              uint16_t hidden_old) {
    y[d] = value;
    if (hidden) hidden[d] = f32_to_f16(f16_to_f32(hidden_old) + f16_to_f32(value));
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
    // the epilogue's operands do not depend on anything computed here: fetch them first
    const bool finisher = threadIdx.x < kPhase2Rows && d0 + threadIdx.x < a.d;
    uint16_t res_bits = 0, hid_bits = 0;
    if (finisher) {
        if (a.residual) res_bits = a.residual[d0 + threadIdx.x];
        if (a.hidden) hid_bits = a.hidden[d0 + threadIdx.x];
    }
    if (!io_ready(a.io_status)) {  // moe.metal:1032-1035
        if (finisher) phase2_finish(a.y, a.hidden, d0 + threadIdx.x, res_bits, hid_bits);
        return;
    }
    const uint32_t cpr = a.f * BITS / 128u, groups = a.f / kGroup, row_bytes = cpr * 16u;
    const bool packed = cpr < 64u && (64u % cpr) == 0u;
    const uint32_t rpl = packed ? min(64u / cpr, kPhase2Rows) : 1u;  // rows per wave load
    const uint32_t seg = packed ? cpr : 64u;
    const uint32_t sub = packed ? lane / cpr : 0u, col = packed ? lane % cpr : lane;
    const bool lane_on = sub < rpl;

    uint32_t cell = a.resolved[k];
    const float wk = f16_to_f32(a.routing_w[k]);
    if (cell == kSentinel && a.fallback) cell = a.fallback[k];  // moe.metal:1037-1038
    const bool live = cell != kSentinel;
    const uint8_t *base = cell_base(a.pool, live ? cell : 0u, a.stride);
    const uint16_t *s_all = reinterpret_cast<const uint16_t *>(base + a.off.down_s_off);
    const uint16_t *b_all = reinterpret_cast<const uint16_t *>(base + a.off.down_b_off);

    if (live) {
        const uint32_t n_groups = kPhase2Rows / rpl;
        typename C::X x[NCH];
        float xs[NCH];
        bool have_x = false;
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
            if (!have_x) {
                load_slices<BITS, NCH>(reinterpret_cast<const uint4 *>(a.acts + size_t(k) * a.f), cpr, col, lane_on, x, xs);
                have_x = true;
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
    if (finisher) {
        float acc = a.residual ? f16_to_f32(res_bits) : 0.0f;
        for (uint32_t i = 0; i < a.top_k; ++i) acc += partial[i][threadIdx.x];
        phase2_finish(a.y, a.hidden, d0 + threadIdx.x, f32_to_f16(acc), hid_bits);
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

constexpr int kPhase1RowPairs = 4;  // (gate, up) row pairs per wave

template <int BITS, int SBITS>
static int launch_phase1(const Phase1Args &a, uint32_t extra_blocks, hipStream_t s) {
    constexpr int RP = kPhase1RowPairs;
    const dim3 grid(a.routed_blocks + extra_blocks), block(256);
    switch (nch_for(a.d, BITS)) {
        case 1: hipLaunchKernelGGL((k_phase1<BITS, 1, RP, SBITS>), grid, block, 0, s, a); break;
        case 2: hipLaunchKernelGGL((k_phase1<BITS, 2, RP, SBITS>), grid, block, 0, s, a); break;
        case 3: hipLaunchKernelGGL((k_phase1<BITS, 3, RP, SBITS>), grid, block, 0, s, a); break;
        default: hipLaunchKernelGGL((k_phase1<BITS, 4, RP, SBITS>), grid, block, 0, s, a); break;
    }
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

static uint32_t phase1_blocks(uint32_t top_k, uint32_t f) {
    const uint32_t waves = (top_k * f + kPhase1RowPairs - 1) / kPhase1RowPairs;
    return (waves + 3) / 4;
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
    const dim3 grid(gemv_blocks(a.rows + a.rows_b, a.n, BITS)), block(256);
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
    const dim3 grid((a.sel.num_experts + 3) / 4), block(256);
    if (router_bits == 0) hipLaunchKernelGGL((k_router<0>), grid, block, 0, s, a);
    else if (router_bits == 8) hipLaunchKernelGGL((k_router<8>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((k_router<4>), grid, block, 0, s, a);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

template <int RK, int BITS>
static void launch_head_nch(const RouterArgs &r, const GemvArgs &g, uint32_t router_blocks, dim3 grid, hipStream_t s) {
    const dim3 block(256);
    switch (nch_for(g.n, BITS)) {
        case 1: hipLaunchKernelGGL((k_head<RK, BITS, 1>), grid, block, 0, s, r, g, router_blocks); break;
        case 2: hipLaunchKernelGGL((k_head<RK, BITS, 2>), grid, block, 0, s, r, g, router_blocks); break;
        case 3: hipLaunchKernelGGL((k_head<RK, BITS, 3>), grid, block, 0, s, r, g, router_blocks); break;
        default: hipLaunchKernelGGL((k_head<RK, BITS, 4>), grid, block, 0, s, r, g, router_blocks); break;
    }
}

// router rows + the shared expert's gate/up rows in one grid
static int launch_head(const RouterArgs &r, uint32_t router_bits, const GemvArgs &g, uint32_t shared_bits,
                       hipStream_t s) {
    const uint32_t router_blocks = (r.sel.num_experts + 3) / 4;
    const dim3 grid(router_blocks + gemv_blocks(g.rows + g.rows_b, g.n, shared_bits));
    if (shared_bits == 4) {
        if (router_bits == 0) launch_head_nch<0, 4>(r, g, router_blocks, grid, s);
        else if (router_bits == 8) launch_head_nch<8, 4>(r, g, router_blocks, grid, s);
        else launch_head_nch<4, 4>(r, g, router_blocks, grid, s);
    } else {
        if (router_bits == 0) launch_head_nch<0, 8>(r, g, router_blocks, grid, s);
        else if (router_bits == 8) launch_head_nch<8, 8>(r, g, router_blocks, grid, s);
        else launch_head_nch<4, 8>(r, g, router_blocks, grid, s);
    }
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

static void fill_select(SelectArgs &sel, const shrike_hip_moe *moe, const void *per_expert_scale,
                        const void *logit_bias, uint32_t num_experts, uint32_t top_k) {
    sel.logits = moe->d_logits;
    sel.per_expert_scale = static_cast<const uint16_t *>(per_expert_scale);
    sel.logit_bias = static_cast<const uint16_t *>(logit_bias);
    sel.num_experts = num_experts; sel.top_k = top_k;
    sel.sigmoid = moe->desc.sigmoid_router_scores; sel.scaling = moe->desc.routed_scaling_factor;
}

static void fill_gemv_gate_up(GemvArgs &a, const shrike_projection *gate, const shrike_projection *up,
                              uint16_t *gate_out, uint16_t *up_out, uint32_t rows, uint32_t n, uint32_t meta,
                              const void *x) {
    a.w_a = static_cast<const uint8_t *>(gate->weights); a.s_a = static_cast<const uint16_t *>(gate->scales);
    a.b_a = static_cast<const uint16_t *>(gate->biases); a.y_a = gate_out;
    a.w_b = static_cast<const uint8_t *>(up->weights); a.s_b = static_cast<const uint16_t *>(up->scales);
    a.b_b = static_cast<const uint16_t *>(up->biases); a.y_b = up_out;
    a.rows = rows; a.rows_b = rows; a.n = n; a.meta = meta;
    a.x = static_cast<const uint16_t *>(x);
}

static void fill_gemv_down(GemvArgs &b, const shrike_projection *down, const uint16_t *gate_in,
                           const uint16_t *up_in, void *h1, uint32_t d, uint32_t f_shared, uint32_t meta,
                           uint32_t act, const void *scalar_gate) {
    b.w_a = static_cast<const uint8_t *>(down->weights); b.s_a = static_cast<const uint16_t *>(down->scales);
    b.b_a = static_cast<const uint16_t *>(down->biases); b.y_a = static_cast<uint16_t *>(h1);
    b.rows = d; b.rows_b = 0; b.n = f_shared; b.meta = meta;
    b.gate_in = gate_in; b.up_in = up_in; b.act = act;
    b.scalar_gate = static_cast<const uint16_t *>(scalar_gate);
}

static int check_shared(const shrike_projection *gate, const shrike_projection *up, const shrike_projection *down,
                        uint32_t bits, uint32_t d, uint32_t f_shared) {
    SHRIKE_REQUIRE(gate && up && down && gate->weights && up->weights && down->weights && gate->scales && gate->biases
                   && up->scales && up->biases && down->scales && down->biases,
                   "sharedExpert: gate, up and down projections must be bound");
    SHRIKE_REQUIRE(bits == 4 || bits == 8, "sharedExpert: bits=%u not in {4, 8}", bits);
    SHRIKE_REQUIRE(d % SHRIKE_GROUP_SIZE == 0 && f_shared % SHRIKE_GROUP_SIZE == 0 && f_shared > 0,
                   "sharedExpert: d=%u and f=%u must be multiples of %u", d, f_shared, SHRIKE_GROUP_SIZE);
    SHRIKE_REQUIRE(nch_for(d, bits) <= 4 && nch_for(f_shared, bits) <= 4, "sharedExpert: rows too long");
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
    a.d = d; a.meta = moe->desc.meta_dtype;
    a.counter = moe->d_counter; a.logits_out = moe->d_logits;
    fill_select(a.sel, moe, d_per_expert_scale, d_logit_bias, num_experts, top_k);
    a.lists.out_indices = d_out_indices;
    a.lists.out_weights = static_cast<uint16_t *>(d_out_weights);
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
    a.routed_blocks = phase1_blocks(top_k, f);
    return bits == 4 ? launch_phase1<4, 0>(a, 0, as_stream(stream)) : launch_phase1<8, 0>(a, 0, as_stream(stream));
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
    if (int rc = check_shared(gate, up, down, bits, d, f_shared)) return rc;
    SHRIKE_REQUIRE(d_x && d_scratch && d_h1, "sharedExpert: x, scratch and h1 must be bound");
    uint16_t *gate_out = static_cast<uint16_t *>(d_scratch), *up_out = gate_out + f_shared;
    GemvArgs a = {};
    fill_gemv_gate_up(a, gate, up, gate_out, up_out, f_shared, d, moe->desc.meta_dtype, d_x);
    if (int rc = bits == 4 ? launch_gemv<4>(a, as_stream(stream)) : launch_gemv<8>(a, as_stream(stream))) return rc;
    GemvArgs b = {};
    fill_gemv_down(b, down, gate_out, up_out, d_h1, d, f_shared, moe->desc.meta_dtype, moe->desc.activation,
                   d_scalar_gate);
    return bits == 4 ? launch_gemv<4>(b, as_stream(stream)) : launch_gemv<8>(b, as_stream(stream));
}

// Three launches: (1) router logit rows + shared gate/up rows; (2) select + classify in the
// prologue of every phase-1 workgroup, the routed gate/up rows, and the shared down rows;
// (3) phase 2 with the shared expert's output as the residual.
int shrike_hip_moe_decode_layer(shrike_hip_moe *moe, void *stream, const shrike_decode_layer_args *g) {
    SHRIKE_REQUIRE(moe != nullptr && g != nullptr, "moe handle or args is NULL");
    const shrike_moe_desc &m = moe->desc;
    if (int rc = check_router(moe, m.num_experts, m.d, m.top_k)) return rc;
    if (int rc = check_offsets(&g->offsets, m.d, m.f, m.routed_weight_bits)) return rc;
    SHRIKE_REQUIRE(g->router_weights && g->effective_scale && g->per_expert_scale && g->logit_bias,
                   "decodeLayer: router operands must be bound");
    SHRIKE_REQUIRE(m.router_weight_bits == 0 || (g->router_scales && g->router_biases),
                   "decodeLayer: affine router needs scales and biases");
    SHRIKE_REQUIRE(g->pool && g->residency && g->x && g->y && g->out_indices && g->out_weights && g->resolved_slots
                   && g->hit_count && g->hit_positions && g->miss_count && g->miss_positions && g->miss_experts
                   && g->acts, "decodeLayer: pool, residency, x, y and the scratch buffers must be bound");
    SHRIKE_REQUIRE(g->pool_slot_stride % 16u == 0, "decodeLayer: pool slot stride must be a multiple of 16");
    hipStream_t s = as_stream(stream);
    const bool shared = g->shared_gate.weights != nullptr;
    const uint32_t sbits = g->shared_bits ? g->shared_bits : m.routed_weight_bits;
    if (shared) {
        if (int rc = check_shared(&g->shared_gate, &g->shared_up, &g->shared_down, sbits, m.d, g->shared_f)) return rc;
        SHRIKE_REQUIRE(g->shared_scratch && g->h1, "decodeLayer: sharedScratch and h1 must be bound");
    }
    uint16_t *gate_out = static_cast<uint16_t *>(g->shared_scratch), *up_out = gate_out ? gate_out + g->shared_f : nullptr;

    RouterArgs r = {};
    r.weights = g->router_weights; r.scales = static_cast<const uint16_t *>(g->router_scales);
    r.biases = static_cast<const uint16_t *>(g->router_biases);
    r.hidden = static_cast<const uint16_t *>(g->x);
    r.effective_scale = static_cast<const uint16_t *>(g->effective_scale);
    r.d = m.d; r.meta = m.meta_dtype; r.counter = moe->d_counter; r.logits_out = moe->d_logits;
    fill_select(r.sel, moe, g->per_expert_scale, g->logit_bias, m.num_experts, m.top_k);
    // the lists stay empty: launch 1 writes logits only

    Phase1Args p1 = {};
    fill_pool(p1.pool, g->pool);
    p1.stride = g->pool_slot_stride; p1.resolved = g->resolved_slots; p1.off = g->offsets;
    p1.x = static_cast<const uint16_t *>(g->x); p1.acts = static_cast<uint16_t *>(g->acts);
    p1.d = m.d; p1.f = m.f; p1.top_k = m.top_k; p1.meta = m.meta_dtype; p1.act = m.activation;
    p1.ebias = m.expert_additive_biases;
    p1.sel = r.sel;
    p1.lists.out_indices = g->out_indices; p1.lists.out_weights = static_cast<uint16_t *>(g->out_weights);
    p1.lists.residency = g->residency; p1.lists.hit_count = g->hit_count; p1.lists.hit_positions = g->hit_positions;
    p1.lists.miss_count = g->miss_count; p1.lists.miss_positions = g->miss_positions;
    p1.lists.miss_experts = g->miss_experts; p1.lists.resolved_slots = g->resolved_slots;
    p1.routed_blocks = phase1_blocks(m.top_k, m.f);

    const void *residual = nullptr;
    bool down_fused = false;
    if (shared) {
        GemvArgs gu = {};
        fill_gemv_gate_up(gu, &g->shared_gate, &g->shared_up, gate_out, up_out, g->shared_f, m.d, m.meta_dtype, g->x);
        if (int rc = launch_head(r, m.router_weight_bits, gu, sbits, s)) return rc;
        fill_gemv_down(p1.shared_down, &g->shared_down, gate_out, up_out, g->h1, m.d, g->shared_f, m.meta_dtype,
                       m.activation, g->shared_scalar_gate);
        down_fused = nch_for(g->shared_f, sbits) == 1;
        residual = g->h1;
    } else {
        if (int rc = launch_router(r, m.router_weight_bits, s)) return rc;  // lists empty: logits only
    }
    const uint32_t extra = down_fused ? gemv_blocks(m.d, g->shared_f, sbits) : 0u;
    int rc;
    if (m.routed_weight_bits == 4)
        rc = !down_fused ? launch_phase1<4, 0>(p1, 0, s) : sbits == 4 ? launch_phase1<4, 4>(p1, extra, s) : launch_phase1<4, 8>(p1, extra, s);
    else
        rc = !down_fused ? launch_phase1<8, 0>(p1, 0, s) : sbits == 4 ? launch_phase1<8, 4>(p1, extra, s) : launch_phase1<8, 8>(p1, extra, s);
    if (rc) return rc;
    if (shared && !down_fused) {
        if (int rc2 = sbits == 4 ? launch_gemv<4>(p1.shared_down, s) : launch_gemv<8>(p1.shared_down, s)) return rc2;
    }

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
