// The group-affine matvec building blocks every decode kernel is made of.
//
// A row of codes is a run of 16-byte chunks; lane l of a 64-wide wave owns column
// chunks l, l+64, ... of every row it touches, so its slice of the activation vector
// sits in registers once (already in the pair layout the fp16 dot wants) and each row
// costs one 128-bit load per chunk. The kernels are bound by memory latency and
// bandwidth: all of a wave's row loads are issued before the first is consumed, and
// out-of-range chunks are clamped to a valid address and zeroed rather than predicated,
// so the loads stay back to back.
#pragma once

#include <type_traits>

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
// The same for a cell every lane of the wave agrees on: the division and the look-up of the
// chunk's base run on the scalar unit (a per-lane index into the argument block would be
// one more dependent memory load ahead of the rows).
__device__ __forceinline__ const uint8_t *cell_base_uniform(const PoolArg &pool, uint32_t cell, uint64_t stride) {
    return cell_base(pool, uint32_t(__builtin_amdgcn_readfirstlane(int(cell))), stride);
}

__device__ __forceinline__ float meta_f32(uint16_t b, uint32_t meta) {
    return meta == SHRIKE_META_F16 ? f16_to_f32(b) : bf16_to_f32(b);
}

// moe.metal:280-288; `act` is uniform, so this is one scalar branch
__device__ __forceinline__ float glu_rt(float g, float u, uint32_t act) {
    if (act == SHRIKE_ACT_SILU) return glu<1>(g, u);
    if (act == SHRIKE_ACT_CLAMPED_SWIGLU) return glu<2>(g, u);
    return glu<0>(g, u);
}

__device__ __forceinline__ float glu_rt_fast(float g, float u, uint32_t act) {
    if (act == SHRIKE_ACT_SILU) return glu_fast<1>(g, u);
    if (act == SHRIKE_ACT_CLAMPED_SWIGLU) return glu_fast<2>(g, u);
    return glu_fast<0>(g, u);
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

// Raw 16-byte pieces of the lane's activation slices for column chunks col + 64*i.
// `off` has bit i set when slice i is not this lane's to use: the load then went to a valid
// stand-in address and unpack_slices zeroes the slice. (Zeroing right behind the load would
// make the wave wait for that load there and then, one load at a time.)
//
// TAIL (4-bit codes): a row of 64 NCH + r chunks with 1 <= r <= 32 ends in a step of half chunks (8 bytes of codes,
// 16 activations) spread over 2 r lanes, in place of a whole step that r lanes would work through and the others
// idle: half chunk 128 NCH + col of the row, for col < 2 r. Bit NCH of `off` marks a lane without one.
template <int BITS, int NCH, bool TAIL = false>
struct SliceRegs {
    uint4 v[NCH][Chunk<BITS>::PIECES];
    uint4 t[2];
    uint32_t off;
};

// whether a row of `cpr` 16-byte chunks is walked as cpr / 64 whole steps and a step of half chunks
inline bool half_chunk_tail(uint32_t cpr, uint32_t bits) { return bits == 4u && cpr > 64u && (cpr % 64u) >= 1u && (cpr % 64u) <= 32u; }

template <int BITS, int NCH, bool TAIL = false>
__device__ __forceinline__ void load_slice_regs(SliceRegs<BITS, NCH, TAIL> &r, const uint4 *vec, uint32_t cpr,
                                                uint32_t col, bool lane_on) {
    typedef Chunk<BITS> C;
    static_assert(!TAIL || BITS == 4, "half chunks are for 4-bit codes");
    r.off = 0u;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const uint32_t c = col + 64u * i;
        const bool on = lane_on && c < cpr;
        const uint32_t cc = on ? c : 0u;
        r.off |= on ? 0u : 1u << i;
#pragma unroll
        for (int j = 0; j < C::PIECES; ++j) r.v[i][j] = vec[cc * C::PIECES + j];
    }
    if (TAIL) {
        const uint32_t h = 128u * NCH + col;
        const bool on = lane_on && h < 2u * cpr;
        const uint32_t hh = on ? h : 0u;
        r.off |= on ? 0u : 1u << NCH;
        r.t[0] = vec[hh * 2u];
        r.t[1] = vec[hh * 2u + 1u];
    }
}

// the activations of a half chunk in the dot's pair layout, and their fp32 sum
struct TailX {
    h2_t p[8];
    float sum;
};

// Pieces -> the dot's pair layout plus the fp32 sum of each slice (for the bias term).
template <int BITS, int NCH, bool TAIL>
__device__ __forceinline__ void unpack_slices(const SliceRegs<BITS, NCH, TAIL> &r, typename Chunk<BITS>::X (&x)[NCH],
                                              float (&xs)[NCH], TailX &xt) {
    typedef Chunk<BITS> C;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < C::PIECES; ++j) {
            const uint4 v = (r.off >> i) & 1u ? zero4() : r.v[i][j];
            C::fill(x[i], j, v);
            s += sum_x8(v);
        }
        xs[i] = s;
    }
    if (TAIL) {
        const bool off = (r.off >> NCH) & 1u;
        const uint4 v0 = off ? zero4() : r.t[0], v1 = off ? zero4() : r.t[1];
        pairs_from_x8(v0, xt.p);
        pairs_from_x8(v1, xt.p + 4);
        xt.sum = sum_x8(v0) + sum_x8(v1);
    }
}
template <int BITS, int NCH>
__device__ __forceinline__ void unpack_slices(const SliceRegs<BITS, NCH, false> &r, typename Chunk<BITS>::X (&x)[NCH],
                                              float (&xs)[NCH]) {
    TailX none;
    unpack_slices<BITS, NCH, false>(r, x, xs, none);
}

template <int BITS, int NCH>
__device__ __forceinline__ void load_slices(const uint4 *vec, uint32_t cpr, uint32_t col, bool lane_on,
                                            typename Chunk<BITS>::X (&x)[NCH], float (&xs)[NCH]) {
    SliceRegs<BITS, NCH> r;
    load_slice_regs<BITS, NCH>(r, vec, cpr, col, lane_on);
    unpack_slices<BITS, NCH>(r, x, xs);
}

// One row's codes and metadata for the lane's column chunks. A chunk that is not this lane's
// is loaded from a valid stand-in address (chunk 0 of the same row) and left as it is: the
// lane's activation slice for it is zero, and so is its term (the row's data being finite).
template <int BITS, int NCH, bool TAIL = false>
struct RowRegs {
    uint4 w[NCH];
    uint16_t s[NCH], b[NCH];
    uint2 tw;  // TAIL: the lane's half chunk of the row, and its group's scale and bias
    uint16_t ts, tb;
};

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// STREAM: the row is read once and by nobody else (a routed expert's rows in decode): the loads are marked
// non-temporal, so that what they bring in does not displace the small tensors every layer call reads again
// (router rows, shared expert, route tables) from the caches behind the compute units.
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

template <int BITS, int NCH, bool STREAM = false, bool TAIL = false>
__device__ __forceinline__ void load_row(RowRegs<BITS, NCH, TAIL> &r, const uint8_t *w_row, const uint16_t *s_row,
                                         const uint16_t *b_row, uint32_t cpr, uint32_t col, bool lane_on) {
    typedef Chunk<BITS> C;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const uint32_t c = col + 64u * i;
        const bool on = lane_on && c < cpr;
        const uint32_t cc = on ? c : 0u;
        const uint32_t g = cc * C::E / kGroup;
        if (STREAM) {
            const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(w_row + 16u * cc));
            r.w[i] = make_uint4(v.x, v.y, v.z, v.w);
            r.s[i] = __builtin_nontemporal_load(s_row + g);
            r.b[i] = __builtin_nontemporal_load(b_row + g);
        } else {
            r.w[i] = *reinterpret_cast<const uint4 *>(w_row + 16u * cc);
            r.s[i] = s_row[g];
            r.b[i] = b_row[g];
        }
    }
    if (TAIL) {
        const uint32_t h = 128u * NCH + col;
        const bool on = lane_on && h < 2u * cpr;
        const uint32_t hh = on ? h : 0u;
        const uint32_t g = hh / 4u;  // sixteen codes a half chunk, 64 a group
        if (STREAM) {
            const u32x2_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t *>(w_row + 8u * hh));
            r.tw = make_uint2(v.x, v.y);
            r.ts = __builtin_nontemporal_load(s_row + g);
            r.tb = __builtin_nontemporal_load(b_row + g);
        } else {
            r.tw = *reinterpret_cast<const uint2 *>(w_row + 8u * hh);
            r.ts = s_row[g];
            r.tb = b_row[g];
        }
    }
}

template <int BITS, int NCH, bool TAIL>
__device__ __forceinline__ float row_partial(const RowRegs<BITS, NCH, TAIL> &r, const typename Chunk<BITS>::X (&x)[NCH],
                                             const float (&xs)[NCH], const TailX &xt, uint32_t meta) {
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        acc = fmaf(meta_f32(r.s[i], meta), Chunk<BITS>::dot(r.w[i], x[i]), acc);
        acc = fmaf(meta_f32(r.b[i], meta), xs[i], acc);
    }
    if (TAIL) {
        float lo, hi;
        dot_word4_first(r.tw.x, xt.p, lo, hi);
        dot_word4(r.tw.y, xt.p + 4, lo, hi);
        acc = fmaf(meta_f32(r.ts, meta), fmaf(lo, 16.0f, hi) * 1048576.0f, acc);
        acc = fmaf(meta_f32(r.tb, meta), xt.sum, acc);
    }
    return acc;
}
template <int BITS, int NCH>
__device__ __forceinline__ float row_partial(const RowRegs<BITS, NCH, false> &r, const typename Chunk<BITS>::X (&x)[NCH],
                                             const float (&xs)[NCH], uint32_t meta) {
    TailX none;
    return row_partial<BITS, NCH, false>(r, x, xs, none, meta);
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

struct NoXSource {  // gemv_job's input is a.x (or the GLU of gate_in and up_in)
    __device__ const uint4 *operator()() const { return nullptr; }
};

// dequant_int4.metal:101-199 / dequant_int8.metal:66-107: y[row] = half(W[row,:] . x), the
// work of workgroup `block` of a grid of 256-thread workgroups.
// x_source(): called by every thread once the rows' own loads are in flight; returns the input row to read
// in place of a.x, or null for a.x (it may first have to produce the row behind a barrier).
template <int BITS, int NCH, class XSource>
__device__ __forceinline__ void gemv_job(const GemvArgs &a, uint32_t block, XSource &&x_source) {
    typedef Chunk<BITS> C;
    const uint32_t lane = threadIdx.x & 63u, wave = wave_index();
    const uint32_t cpr = a.n * BITS / 128u, groups = a.n / kGroup, row_bytes = cpr * 16u;
    const bool packed = NCH == 1 && cpr < 64u && (64u % cpr) == 0u;  // (NCH >= 2: more than 64 chunks a row, known to the instance)
    const uint32_t rpl = packed ? 64u / cpr : 1u;
    const uint32_t seg = packed ? cpr : 64u;
    const uint32_t sub = packed ? lane / cpr : 0u, col = packed ? lane % cpr : lane;
    const uint32_t total = a.rows + a.rows_b;
    const uint32_t first = (block * 4u + wave) * kGemvRowsPerWave * rpl;
    const bool active = first < total;
    // The two row sets' pointers, pinned in scalar registers: picking between the FIELDS of the argument block by a
    // per-lane condition would otherwise become a vector load of the chosen pointer from constant memory, a
    // dependent memory round trip ahead of every row load and every store.
    const uint8_t *w_a = a.w_a, *w_b = a.w_b;
    const uint16_t *s_a = a.s_a, *s_b = a.s_b, *b_a = a.b_a, *b_b = a.b_b;
    uint16_t *y_a = a.y_a, *y_b = a.y_b;
    asm volatile("" : "+s"(w_a), "+s"(w_b), "+s"(s_a), "+s"(s_b), "+s"(b_a), "+s"(b_b), "+s"(y_a), "+s"(y_b));

    // the input slice first: in-order load return must not hold it behind the rows
    SliceRegs<BITS, NCH> xin;
    constexpr bool kPlainX = std::is_same<typename std::decay<XSource>::type, NoXSource>::value;
    if (kPlainX && !a.gate_in && active) load_slice_regs<BITS, NCH>(xin, reinterpret_cast<const uint4 *>(a.x), cpr, col, true);
    uint16_t gate_bits = 0;
    if (a.scalar_gate) gate_bits = a.scalar_gate[0];

    RowRegs<BITS, NCH> rows[kGemvRowsPerWave];
    uint32_t row[kGemvRowsPerWave];
    bool on[kGemvRowsPerWave];
    if (active) {
#pragma unroll
        for (uint32_t j = 0; j < kGemvRowsPerWave; ++j) {
            row[j] = first + j * rpl + sub;
            on[j] = row[j] < total;
            const uint32_t rr = on[j] ? row[j] : 0u;
            const bool second = rr >= a.rows;
            const uint32_t local = second ? rr - a.rows : rr;
            load_row<BITS, NCH>(rows[j], (second ? w_b : w_a) + size_t(local) * row_bytes,
                                (second ? s_b : s_a) + size_t(local) * groups,
                                (second ? b_b : b_a) + size_t(local) * groups, cpr, col, on[j]);
        }
    }
    if (!kPlainX) {
        const uint4 *x_row = x_source();
        if (active) load_slice_regs<BITS, NCH>(xin, x_row, cpr, col, true);
    } else if (a.gate_in) {
        // dequant_int4.metal:283-287: act = half(glu(gate, up)) once per workgroup, staged in LDS; a thread takes
        // pairs of neighbours, so that a short row still spreads over the whole workgroup
        __shared__ uint4 act_l[SHRIKE_MAX_HIDDEN / 8];
        uint32_t *act_w = reinterpret_cast<uint32_t *>(act_l);
        for (uint32_t p = threadIdx.x; p < a.n / 2u; p += 256u) {
            const uint32_t gw = reinterpret_cast<const uint32_t *>(a.gate_in)[p];
            const uint32_t uw = reinterpret_cast<const uint32_t *>(a.up_in)[p];
            const uint16_t lo = f32_to_f16(glu_rt(f16_to_f32(uint16_t(gw)), f16_to_f32(uint16_t(uw)), a.act));
            const uint16_t hi = f32_to_f16(glu_rt(f16_to_f32(uint16_t(gw >> 16)), f16_to_f32(uint16_t(uw >> 16)), a.act));
            act_w[p] = uint32_t(lo) | (uint32_t(hi) << 16);
        }
        __syncthreads();
        if (active) load_slice_regs<BITS, NCH>(xin, act_l, cpr, col, true);
    }
    if (!active) return;
    typename C::X x[NCH];
    float xs[NCH];
    unpack_slices<BITS, NCH>(xin, x, xs);
    // what the rows' epilogue shares is formed once: the gate's divisor, and the segment's last lane by a mask
    // (a segment is a power of two lanes)
    const bool gated = a.scalar_gate != nullptr;
    const float gate_div = gated ? 1.0f + expf(-f16_to_f32(gate_bits)) : 1.0f;
    const bool writer_lane = (lane & (seg - 1u)) == seg - 1u;
    float sums[kGemvRowsPerWave];
#pragma unroll
    for (uint32_t j = 0; j < kGemvRowsPerWave; ++j) sums[j] = row_partial<BITS, NCH>(rows[j], x, xs, a.meta);
#pragma unroll
    for (uint32_t j = 0; j < kGemvRowsPerWave; ++j) sums[j] = seg_sum(sums[j], seg);  // four independent chains
#pragma unroll
    for (uint32_t j = 0; j < kGemvRowsPerWave; ++j) {
        if (on[j] && writer_lane) {
            const bool second = row[j] >= a.rows;
            uint16_t yh = f32_to_f16(sums[j]);
            if (gated) yh = f32_to_f16(f16_to_f32(yh) / gate_div);
            (second ? y_b : y_a)[second ? row[j] - a.rows : row[j]] = yh;
        }
    }
}

template <int BITS, int NCH>
__device__ __forceinline__ void gemv_job(const GemvArgs &a, uint32_t block) {
    gemv_job<BITS, NCH>(a, block, NoXSource{});
}

inline uint32_t nch_for(uint32_t n, uint32_t bits) { return (n * bits / 128u + 63u) / 64u; }

inline uint32_t gemv_blocks(uint32_t total_rows, uint32_t n, uint32_t bits) {
    const uint32_t cpr = n * bits / 128u;
    const uint32_t rpl = (cpr < 64u && 64u % cpr == 0u) ? 64u / cpr : 1u;
    const uint32_t per_wave = kGemvRowsPerWave * rpl;
    return ((total_rows + per_wave - 1) / per_wave + 3) / 4;
}

inline void fill_pool(PoolArg &p, const shrike_pool_bases *pool) {
    for (uint32_t i = 0; i < SHRIKE_POOL_MAX_CHUNKS; ++i) p.base[i] = static_cast<const uint8_t *>(pool->base[i]);
    p.cells_per_chunk = pool->cells_per_chunk ? pool->cells_per_chunk : 1u;
}

// ------------------------------------------------------------ routing

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

__device__ __forceinline__ float sigmoidf_(float v) { return 1.0f / (1.0f + expf(-v)); }
// The selection score of one expert (moe.metal:436-440) as an unsigned key: a larger score is a larger key, 0 marks
// what can never be taken (NaN and -inf; the reference's slots start at -inf, index 0).
__device__ __forceinline__ uint32_t score_key(float raw, float bias, uint32_t sigmoid) {
    float s = (sigmoid ? sigmoidf_(raw) : raw) + bias;
    s = s + 0.0f;  // -0 and +0 tie
    const uint32_t u = __float_as_uint(s);
    const uint32_t ord = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
    return (s == s && s > -INFINITY) ? ord : 0u;
}
__device__ __forceinline__ float key_score(uint32_t key) {
    return key == 0u ? -INFINITY : __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}

template <bool COHERENT>
__device__ __forceinline__ float load_logit(const float *p) {
    return COHERENT ? __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : *p;
}

// moe.metal:419-491 and :121-151, run by one wave. Lane l holds experts l, l+64, l+128,
// l+192 with their bias, scale and residency word (all fetched up front, so nothing that
// follows waits on memory). Each of the top_k rounds takes the wave-wide maximum score and,
// among the experts that hold it, the lowest index (moe.metal:443-449); a NaN score is never
// taken, and -inf scores are never taken either (the reference's slots start at -inf, index
// 0). On return lane p < top_k holds position p's resolved cell (sentinel on a miss).
// COHERENT reads the logits past the non-coherent caches (they were written by other
// workgroups of the same launch); otherwise they come from an earlier launch.
// One wave's table of candidates in LDS for route_wave (a workgroup whose waves route side
// by side gives each its own).
struct RouteScratch {
    uint32_t key[256], gain[256], cellv[256];
    float raw[256];
};

__device__ __forceinline__ void finish_routes(const SelectArgs &a, const RouteLists &out, uint32_t lane, bool write_lists,
                                              uint32_t mine, uint32_t my_key, float my_raw, float my_gain,
                                              uint32_t cell_of_mine, uint32_t &my_cell);

template <bool COHERENT>
__device__ void route_wave(const SelectArgs &a, const RouteLists &out, uint32_t lane, bool write_lists,
                           uint32_t &my_cell, RouteScratch &lds) {
    // key = the score's bits mapped to an unsigned order (larger score, larger key); 0 marks
    // what can never be taken: NaN, -inf and experts past num_experts
    uint32_t key[4], cellv[4], gainv[4];
    float raw[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t e = lane + 64u * j;
        const bool on = e < a.num_experts;
        const uint32_t ee = on ? e : 0u;
        raw[j] = load_logit<COHERENT>(a.logits + ee);
        const float bias = bf16_to_f32(a.logit_bias[ee]);
        gainv[j] = a.per_expert_scale[ee];
        const uint64_t word = out.residency ? out.residency[ee] : 0;
        // moe.metal:136-146: a hit names its cell, anything else is the sentinel
        cellv[j] = (uint32_t(word >> 32) == SHRIKE_RESIDENCY_RESIDENT) ? uint32_t(word) : kSentinel;
        key[j] = on ? score_key(raw[j], bias, a.sigmoid) : 0u;
    }
    const uint32_t K = a.top_k;
    // Every lane parks its four candidates in LDS; after the rounds lane p fetches position
    // p's full key, gain, cell (and raw logit) by expert index with one read each.
    uint32_t *s_key = lds.key, *s_gain = lds.gain, *s_cellv = lds.cellv;
    float *s_raw = lds.raw;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        s_key[lane + 64u * j] = key[j];
        s_gain[lane + 64u * j] = gainv[j];
        s_cellv[lane + 64u * j] = cellv[j];
        if (a.sigmoid) s_raw[lane + 64u * j] = raw[j];
    }
    // Fast rounds on a 32-bit composite key: the score key's upper 24 bits over 255 - index.
    // One wave-wide max per round names the winner (higher score, lower index on equal
    // scores). The composite order is the true order unless two candidates agree in those 24
    // bits and differ below them; that is checked once after the rounds, and the exact rounds
    // further down run instead if it can have mattered.
    uint32_t ck[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) ck[j] = key[j] ? ((key[j] & 0xffffff00u) | (255u - (lane + 64u * j))) : 0u;
    uint32_t fast_top = 0;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        if (uint32_t(r) < K) {
            const uint32_t best = max(max(ck[0], ck[1]), max(ck[2], ck[3]));
            const uint32_t top = wave_max_u32(best);  // 0: nothing left to take
#pragma unroll
            for (int j = 0; j < 4; ++j) ck[j] = ck[j] == top ? 0u : ck[j];
            fast_top = lane == uint32_t(r) ? top : fast_top;
        }
    }
    // The fast result is the true one when (a) the winners' prefixes fall strictly from rank
    // to rank (equal prefixes are fine only for equal full keys, where the index decided), and
    // (b) no candidate left behind shares the last winner's prefix with a different full key.
    uint32_t mine = fast_top ? 255u - (fast_top & 255u) : 0u;
    uint32_t my_key = fast_top ? s_key[mine] : 0u;
    const uint32_t next_top = __shfl_down(fast_top, 1), next_key = __shfl_down(my_key, 1);
    const bool pair_clash = lane + 1u < K && next_top != 0u && (fast_top >> 8) == (next_top >> 8) && my_key != next_key;
    const uint32_t last_top = uint32_t(__builtin_amdgcn_readlane(int(fast_top), int(K) - 1));
    const uint32_t last_key = uint32_t(__builtin_amdgcn_readlane(int(my_key), int(K) - 1));
    bool left_clash = false;
#pragma unroll
    for (int j = 0; j < 4; ++j) left_clash |= ck[j] != 0u && last_top != 0u && (ck[j] >> 8) == (last_top >> 8) && key[j] != last_key;
    if (__ballot(pair_clash || left_clash) != 0) {
        // exact rounds: wave-wide max of the full key, then the lowest index among its holders
        mine = 0; my_key = 0;
#pragma unroll 1
        for (uint32_t r = 0; r < K; ++r) {
            uint32_t best = key[0], bj = 0;
#pragma unroll
            for (int j = 1; j < 4; ++j) {
                const bool better = key[j] > best;  // strict: the lower index of equals stays
                best = better ? key[j] : best;
                bj = better ? uint32_t(j) : bj;
            }
            const uint32_t top = wave_max_u32(best);
            uint32_t win = 0;
            if (top != 0u) {
                const bool holds = best == top;
                win = wave_min_u32(holds ? lane + 64u * bj : 0xffffffffu);
                const bool me = lane == (win & 63u);
#pragma unroll
                for (int j = 0; j < 4; ++j) key[j] = (me && (win >> 6) == uint32_t(j)) ? 0u : key[j];
            }
            if (lane == r) { mine = win; my_key = top; }
        }
    }
    const float my_gain = bf16_to_f32(uint16_t(s_gain[mine]));
    const uint32_t cell_of_mine = s_cellv[mine];
    finish_routes(a, out, lane, write_lists, mine, my_key, a.sigmoid ? s_raw[mine] : 0.0f, my_gain, cell_of_mine, my_cell);
}

// The second half of the select (moe.metal:460-490) and the classification (moe.metal:121-151) for a wave whose lane
// p < top_k holds position p's expert `mine`, its score key, raw logit, gain and residency-resolved cell.
__device__ __forceinline__ void finish_routes(const SelectArgs &a, const RouteLists &out, uint32_t lane, bool write_lists,
                                              uint32_t mine, uint32_t my_key, float my_raw, float my_gain,
                                              uint32_t cell_of_mine, uint32_t &my_cell) {
    const uint32_t K = a.top_k;
    const float my_score = key_score(my_key);
    const bool on = lane < K;
    float weight;
    if (a.sigmoid) {  // moe.metal:460-474
        const float orig = on ? sigmoidf_(my_raw) : 0.0f;
        float sum = 0.0f;
#pragma unroll
        for (int r = 0; r < 8; ++r) {  // rank order, as the reference adds them
            const float o = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(orig), r));
            if (uint32_t(r) < K) sum += o;
        }
        weight = orig * (a.scaling / (sum + 1e-20f));
    } else {  // moe.metal:477-490
        const float top = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_score), 0));
        const float ex = on ? expf(my_score - top) : 0.0f;
        float sum = 0.0f;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const float o = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(ex), r));
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
    const bool hit = on && cell_of_mine != kSentinel;
    if (hit) my_cell = cell_of_mine;
    if (!write_lists) return;
    if (out.hit_count == nullptr) {  // a batch of tokens: the cells alone, no hit and miss lists
        if (on) out.resolved_slots[lane] = hit ? cell_of_mine : kSentinel;
        return;
    }
    const uint64_t hit_mask = __ballot(hit), miss_mask = __ballot(on && !hit);
    const uint64_t below = (uint64_t(1) << lane) - 1u;
    if (hit) {
        out.hit_positions[__popcll(hit_mask & below)] = lane;
        out.resolved_slots[lane] = cell_of_mine;
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

// ---- the route table of the fused layer
//
// The layer's first launch leaves one 16-byte entry per expert: everything the selection needs, already combined
// (score key with the bias folded in, the cell the residency word resolves to, the raw logit and the gain). The
// second launch's waves then select from 4 KB written a moment ago instead of gathering four cold per-layer
// arrays, and need no arithmetic before the first comparison.
struct RouteEntry {
    uint32_t key, cell;
    float raw;
    uint32_t gain;  // bf16 bits of per_expert_scale
};

__device__ __forceinline__ void write_route_entry(RouteEntry *table, uint32_t e, float raw, uint16_t bias_bits,
                                                  uint16_t gain_bits, uint64_t word, uint32_t sigmoid) {
    uint4 v;
    v.x = score_key(raw, bf16_to_f32(bias_bits), sigmoid);
    // moe.metal:136-146: a hit names its cell, anything else is the sentinel
    v.y = (uint32_t(word >> 32) == SHRIKE_RESIDENCY_RESIDENT) ? uint32_t(word) : kSentinel;
    v.z = __float_as_uint(raw);
    v.w = gain_bits;
    *reinterpret_cast<uint4 *>(table + e) = v;
}

// What the select leaves in a wave: lane p < top_k holds position p's expert and its entry.
struct TableSelect {
    uint32_t mine, my_key, my_cell, my_gain;
    float my_raw;
};

// moe.metal:419-458 over the route table, by one wave, all in registers. Lane l holds experts 4l .. 4l+3 and first
// sorts its four by key, descending, equals in index order (exchanges of neighbours only, so the sort is stable). A
// round then looks at the heads alone: the wave's maximum, the ballot of the lanes whose head holds it, the lowest
// such lane (the lowest index, moe.metal:443-449), whose head's entry is read across by lane index and popped. The
// full 32-bit key is compared, so the order is exact. Positions that find nothing left take expert 0 with score
// -inf, as the reference's initial slots do.
// last_round (uniform): the last position the caller needs; later rounds are skipped.
// Up to 64 experts: lane l holds expert l alone, so there is nothing to sort and a round pops by clearing one key.
__device__ __forceinline__ TableSelect select_from_small_table(const RouteEntry *table, uint32_t num_experts, uint32_t K,
                                                               uint32_t lane, uint32_t last_round) {
    const uint4 v = reinterpret_cast<const uint4 *>(table)[lane];
    uint32_t key = lane < num_experts ? v.x : 0u;
    TableSelect r;
    r.mine = 0; r.my_key = 0;
    r.my_cell = uint32_t(__builtin_amdgcn_readfirstlane(int(v.y)));
    r.my_gain = uint32_t(__builtin_amdgcn_readfirstlane(int(v.w)));
    r.my_raw = __uint_as_float(uint32_t(__builtin_amdgcn_readfirstlane(int(v.z))));
#pragma unroll
    for (int round = 0; round < 8; ++round) {
        if (uint32_t(round) < K && uint32_t(round) <= last_round) {
            const uint32_t top = wave_max_u32(key);
            if (top != 0u) {  // uniform
                const int win = __ffsll((long long)__ballot(key == top)) - 1;
                const uint32_t wcell = uint32_t(__builtin_amdgcn_readlane(int(v.y), win));
                const uint32_t wraw = uint32_t(__builtin_amdgcn_readlane(int(v.z), win));
                const uint32_t wgain = uint32_t(__builtin_amdgcn_readlane(int(v.w), win));
                key = lane == uint32_t(win) ? 0u : key;
                if (lane == uint32_t(round)) {
                    r.mine = uint32_t(win); r.my_key = top; r.my_cell = wcell; r.my_gain = wgain;
                    r.my_raw = __uint_as_float(wraw);
                }
            }
        }
    }
    return r;
}

__device__ __forceinline__ TableSelect select_from_table(const RouteEntry *table, uint32_t num_experts, uint32_t K,
                                                         uint32_t lane, uint32_t last_round) {
    if (num_experts <= 64u) return select_from_small_table(table, num_experts, K, lane, last_round);
    uint32_t key[4], cellv[4], rawv[4], gainv[4], idx[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint4 v = reinterpret_cast<const uint4 *>(table)[lane * 4u + j];
        idx[j] = lane * 4u + j;
        key[j] = idx[j] < num_experts ? v.x : 0u;
        cellv[j] = v.y; rawv[j] = v.z; gainv[j] = v.w;
    }
    TableSelect r;
    // what a position with nothing left to take names: expert 0
    r.mine = 0; r.my_key = 0;
    r.my_cell = uint32_t(__builtin_amdgcn_readfirstlane(int(cellv[0])));
    r.my_gain = uint32_t(__builtin_amdgcn_readfirstlane(int(gainv[0])));
    r.my_raw = __uint_as_float(uint32_t(__builtin_amdgcn_readfirstlane(int(rawv[0]))));
    auto exchange = [&](int a, int b) {  // neighbours a < b: the later one moves ahead only when strictly larger
        const bool swap = key[b] > key[a];
        uint32_t t;
        t = key[a]; key[a] = swap ? key[b] : t; key[b] = swap ? t : key[b];
        t = cellv[a]; cellv[a] = swap ? cellv[b] : t; cellv[b] = swap ? t : cellv[b];
        t = idx[a]; idx[a] = swap ? idx[b] : t; idx[b] = swap ? t : idx[b];
        t = rawv[a]; rawv[a] = swap ? rawv[b] : t; rawv[b] = swap ? t : rawv[b];
        t = gainv[a]; gainv[a] = swap ? gainv[b] : t; gainv[b] = swap ? t : gainv[b];
    };
    exchange(0, 1); exchange(2, 3); exchange(1, 2); exchange(0, 1); exchange(2, 3); exchange(1, 2);
#pragma unroll
    for (int round = 0; round < 8; ++round) {
        if (uint32_t(round) < K && uint32_t(round) <= last_round) {
            const uint32_t top = wave_max_u32(key[0]);
            if (top != 0u) {  // uniform
                const int win = __ffsll((long long)__ballot(key[0] == top)) - 1;
                const uint32_t widx = uint32_t(__builtin_amdgcn_readlane(int(idx[0]), win));
                const uint32_t wcell = uint32_t(__builtin_amdgcn_readlane(int(cellv[0]), win));
                const uint32_t wraw = uint32_t(__builtin_amdgcn_readlane(int(rawv[0]), win));
                const uint32_t wgain = uint32_t(__builtin_amdgcn_readlane(int(gainv[0]), win));
                const bool me = lane == uint32_t(win);
#pragma unroll
                for (int j = 0; j < 3; ++j) {
                    key[j] = me ? key[j + 1] : key[j];
                    cellv[j] = me ? cellv[j + 1] : cellv[j];
                    idx[j] = me ? idx[j + 1] : idx[j];
                    rawv[j] = me ? rawv[j + 1] : rawv[j];
                    gainv[j] = me ? gainv[j + 1] : gainv[j];
                }
                key[3] = me ? 0u : key[3];
                if (lane == uint32_t(round)) {
                    r.mine = widx; r.my_key = top; r.my_cell = wcell; r.my_gain = wgain;
                    r.my_raw = __uint_as_float(wraw);
                }
            }
        }
    }
    return r;
}

}  // namespace shrike
