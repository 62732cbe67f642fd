// The grouped expert FFN of prefill for gfx950 (PrefillGroupedRoutedMoE.encodeGroupedExpertGEMMs,
// PrefillGroupedRoutedMoE.swift:925-1126): for every 64-row tile of one expert's pairs,
// act = fp16(glu(gate . X, up . X)) and partial = fp16(down . act), on the matrix cores.
//
// The quantised weights never become fp16 weights. With w = q * s + b per group of 64,
//   sum_k x_k w_k = sum_g s_g (sum_{k in g} x_k q_k) + sum_g b_g (sum_{k in g} x_k),
// the codes enter v_mfma_f32_32x32x16_f16 as they are: a 4- or 8-bit code placed in the low
// bits of an fp16 is the subnormal q * 2^-24, which the matrix core multiplies exactly, so
// the per-group product sum_k x_k q_k comes out of four chained MFMAs in fp32 and is scaled
// by s_g * 2^24 on the vector ALU. The bias term is one more short matrix product between
// the per-row group sums of X (fp32 sums carried as fp16 hi + lo, see k_row_group_sums) and
// the group biases.
#include "decode_launch.h"
#include "prefill_common.h"

#include "../../include/shrike_host.h"

#include <type_traits>

namespace shrike {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr uint32_t kChunkK = 256;                 // k staged in LDS per step: four groups
constexpr uint32_t kGroupsPerChunk = kChunkK / 64;
constexpr uint32_t kStagePieces = kChunkK / 8;     // 16-byte pieces of one staged row
constexpr uint32_t kStageRows = 256 / kStagePieces; // rows one pass of the workgroup stages
constexpr uint32_t kStagePasses = kRowTile / kStageRows;
constexpr uint32_t kLdsRow = kChunkK + 8;         // halves per staged row; the pad spreads the banks
static_assert(kRowTile == 64, "a row tile is one or two 32-row MFMA tiles");
constexpr float kTwo24 = 16777216.0f;

struct FfnArgs {
    PoolArg pool;
    uint64_t stride;
    shrike_expert_offsets off;
    const shrike_row_tile *tiles;
    const uint32_t *tile_count;
    const uint64_t *residency;    // null, or the table that names the tiles' cells at this call
    uint32_t pair_lo, pair_hi;    // the sorted pairs this call covers; rows of other pairs are left alone
    const shrike_token_expert_pair *pairs;
    const uint16_t *hidden;       // fp16[T, hidden_stride]
    uint32_t hidden_stride;
    const uint32_t *hidden_sums;  // (hi, lo)[T, d / 64]
    uint16_t *act;                // fp16[tiles * 64, f]
    const uint32_t *act_sums;     // (hi, lo)[tiles * 64, f / 64]
    uint16_t *partials;           // fp16[T * top_k, d]
    uint32_t d, f, top_k, meta, act_kind, ebias;
    // dense mode (one resident FFN over all rows, the shared expert): the three projections as
    // separate tensors, rows in token order, output row = token
    const uint8_t *dense_w[3];
    const uint16_t *dense_s[3], *dense_b[3];
    uint32_t dense_rows;
    uint32_t round_gate_up;        // gate and up pass through fp16 before the GLU (dequant_int4.metal:206-287)
    const uint16_t *scalar_gate;   // fp16[rows] or null: row m's output * sigmoid(gate[m]) (moe.metal:1195-1207)
    uint32_t resident_workgroups;  // workgroups of these kernels the device holds at once (two a compute unit)
};

union Frag {
    half8 h;
    uint32_t u[4];
    uint4 v;
};

// 4-bit: the eight codes of one word as fp16 subnormals in the order (0,4,1,5,2,6,3,7),
// which is the order the staged A rows are permuted to.
__device__ __forceinline__ half8 codes4(uint32_t w) {
    Frag f;
    f.u[0] = w & 0x000f000fu;
    f.u[1] = (w >> 4) & 0x000f000fu;
    f.u[2] = (w >> 8) & 0x000f000fu;
    f.u[3] = (w >> 12) & 0x000f000fu;
    return f.h;
}
// 8-bit: eight codes of two words, in order
__device__ __forceinline__ half8 codes8(uint32_t w0, uint32_t w1) {
    Frag f;
    f.u[0] = __builtin_amdgcn_perm(0u, w0, 0x0c010c00u);
    f.u[1] = __builtin_amdgcn_perm(0u, w0, 0x0c030c02u);
    f.u[2] = __builtin_amdgcn_perm(0u, w1, 0x0c010c00u);
    f.u[3] = __builtin_amdgcn_perm(0u, w1, 0x0c030c02u);
    return f.h;
}

template <int BITS>
struct BRegs {  // one lane's codes of one weight row for one group: its 32 k
    uint4 w[BITS / 4];
    uint16_t scale;
};

// row_s == nullptr: the codes alone (the caller has the scale already)
template <int BITS>
__device__ __forceinline__ void load_b(BRegs<BITS> &r, const uint8_t *row_w, const uint16_t *row_s, uint32_t g, uint32_t kb) {
    const uint4 *p = reinterpret_cast<const uint4 *>(row_w + size_t(g) * (kGroup * BITS / 8) + kb * (4 * BITS));
#pragma unroll
    for (int i = 0; i < BITS / 4; ++i) r.w[i] = p[i];
    if (row_s) r.scale = row_s[g];
}

template <int BITS>
__device__ __forceinline__ half8 b_step(const BRegs<BITS> &r, int s) {
    if (BITS == 4) {
        const uint32_t w[4] = {r.w[0].x, r.w[0].y, r.w[0].z, r.w[0].w};
        return codes4(w[s]);
    } else {
        const uint32_t w[8] = {r.w[0].x, r.w[0].y, r.w[0].z, r.w[0].w, r.w[BITS / 4 - 1].x, r.w[BITS / 4 - 1].y, r.w[BITS / 4 - 1].z, r.w[BITS / 4 - 1].w};
        return codes8(w[2 * s], w[2 * s + 1]);
    }
}

// MODE 0: gate and up rows n0..n0+31 of one expert against the gathered token rows, GLU,
// fp16 activations out. MODE 1: down rows n0..n0+63 against the activations, fp16 partials
// scattered to (token, rank).
// One row tile against one block of weight rows. MT = the tile's 32-row MFMA tiles, a template
// parameter so that the main loop is straight-line code: the compiler is then free to put one
// chain's matrix instructions beside another chain's vector work.
// MODE 0 leaves its activations through LDS: whole 16-byte pieces of a row go out together, and the group sums of the
// tile's rows that the down product's bias term needs are formed here, in k_row_group_sums' order of additions (eight
// lanes a group, a lane adds its eight values in order, the partial sums fold pairwise), instead of by a launch of
// their own between the two products. Every wave of the workgroup stays to the end for the barriers.
// META: the type of the scales and biases (SHRIKE_META_*), known to the instance so that a scale converts one way.
template <int BITS, int MODE, bool DENSE, uint32_t MT, int META>
__device__ __forceinline__ void ffn_tile(const FfnArgs &a, const shrike_row_tile &tile, uint32_t tile_index, uint32_t col_block,
                                         uint16_t (&s_a)[2][kRowTile][kLdsRow]) {
    const uint32_t K = MODE == 0 ? a.d : a.f, N = MODE == 0 ? a.f : a.d;
    const uint32_t G = K / kGroup;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t col = lane & 31u, kb = lane >> 5;
    const uint32_t n0 = (col_block * 4u + wave) * (MODE == 0 ? 32u : 64u);
    const bool active = n0 < N;

    // ---- A staging: thread -> (row = tid / kStagePieces + kStageRows i, 16-byte piece = tid % kStagePieces)
    const uint32_t piece = threadIdx.x % kStagePieces, row0 = threadIdx.x / kStagePieces;
    const uint16_t *src_row[kStagePasses];
#pragma unroll
    for (uint32_t i = 0; i < kStagePasses; ++i) {
        const uint32_t r = min(row0 + kStageRows * i, tile.rows - 1u);  // rows past the tile repeat its last row
        if (MODE == 0) {
            const uint32_t token = DENSE ? tile.pair_start + r : a.pairs[tile.pair_start + r].token;
            src_row[i] = a.hidden + size_t(token) * a.hidden_stride;
        } else {
            src_row[i] = a.act + (size_t(tile_index) * kRowTile + r) * a.f;
        }
    }
    uint4 stage[kStagePasses];
    auto fetch = [&](uint32_t chunk) {
        const uint32_t k = chunk * kChunkK + piece * 8u;
#pragma unroll
        for (uint32_t i = 0; i < kStagePasses; ++i)
            if (i * kStageRows < MT * 32u && k < K) stage[i] = *reinterpret_cast<const uint4 *>(src_row[i] + k);
    };
    auto commit = [&](uint32_t buf) {
#pragma unroll
        for (uint32_t i = 0; i < kStagePasses; ++i) {
            if (i * kStageRows >= MT * 32u) continue;
            uint4 v = stage[i];
            if (BITS == 4) {  // (0,1,2,3,4,5,6,7) -> (0,4,1,5,2,6,3,7), to meet codes4
                uint4 p;
                p.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
                p.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
                p.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
                p.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
                v = p;
            }
            *reinterpret_cast<uint4 *>(&s_a[buf][row0 + kStageRows * i][piece * 8u]) = v;
        }
    };

    // ---- B rows of this lane
    const uint8_t *base = DENSE ? nullptr : cell_base(a.pool, tile.cell, a.stride);
    const uint32_t row_bytes = K * BITS / 8u;
    const uint8_t *bw[2];
    const uint16_t *bs[2], *bb[2];
    {
        const uint32_t n = active ? n0 + col : 0u;
        if (DENSE) {
            const int first = MODE == 0 ? 0 : 2, second = MODE == 0 ? 1 : 2;
            const uint32_t n1 = MODE == 0 ? n : n + 32u;
            bw[0] = a.dense_w[first] + size_t(n) * row_bytes;
            bw[1] = a.dense_w[second] + size_t(n1) * row_bytes;
            bs[0] = a.dense_s[first] + size_t(n) * G;
            bs[1] = a.dense_s[second] + size_t(n1) * G;
            bb[0] = a.dense_b[first] + size_t(n) * G;
            bb[1] = a.dense_b[second] + size_t(n1) * G;
        } else if (MODE == 0) {
            bw[0] = base + a.off.gate_w_off + size_t(n) * row_bytes;
            bw[1] = base + a.off.up_w_off + size_t(n) * row_bytes;
            bs[0] = reinterpret_cast<const uint16_t *>(base + a.off.gate_s_off) + size_t(n) * G;
            bs[1] = reinterpret_cast<const uint16_t *>(base + a.off.up_s_off) + size_t(n) * G;
            bb[0] = reinterpret_cast<const uint16_t *>(base + a.off.gate_b_off) + size_t(n) * G;
            bb[1] = reinterpret_cast<const uint16_t *>(base + a.off.up_b_off) + size_t(n) * G;
        } else {
            const uint32_t n1 = n + 32u;
            bw[0] = base + a.off.down_w_off + size_t(n) * row_bytes;
            bw[1] = base + a.off.down_w_off + size_t(n1) * row_bytes;
            bs[0] = reinterpret_cast<const uint16_t *>(base + a.off.down_s_off) + size_t(n) * G;
            bs[1] = reinterpret_cast<const uint16_t *>(base + a.off.down_s_off) + size_t(n1) * G;
            bb[0] = reinterpret_cast<const uint16_t *>(base + a.off.down_b_off) + size_t(n) * G;
            bb[1] = reinterpret_cast<const uint16_t *>(base + a.off.down_b_off) + size_t(n1) * G;
        }
    }

    f32x16 total[2][MT];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (uint32_t mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 16; ++i) total[nt][mt][i] = 0.0f;

    // the rows' group sums for the bias term: their addresses hang on the pair records, so they are
    // worked out here, far ahead of their use
    const uint32_t *sums = MODE == 0 ? a.hidden_sums : a.act_sums;
    const uint32_t *sum_row[MT];
#pragma unroll
    for (uint32_t mt = 0; mt < MT; ++mt) {
        const uint32_t r = min(mt * 32u + col, tile.rows - 1u);
        const uint32_t token = (MODE != 0) ? 0u : DENSE ? tile.pair_start + r : a.pairs[tile.pair_start + r].token;
        sum_row[mt] = MODE == 0 ? sums + size_t(token) * G : sums + (size_t(tile_index) * kRowTile + r) * G;
    }

    // A row's scales for the four groups of a staged chunk are one aligned 8-byte run when G is a
    // multiple of 4: they are then fetched a chunk ahead with one load instead of four two-byte ones
    // (every such load costs a cache-line look-up per lane, as each lane reads a row of its own).
    // Decided from the tensors' start (the same for every lane, a row's scales being G * 2 bytes), so
    // that the choice is uniform over the workgroup and each variant of the loop is straight-line code.
    static_assert(kGroupsPerChunk == 4, "a chunk's scales are read as four 16-bit values");
    const uint32_t scale_misalign = uint32_t((reinterpret_cast<uintptr_t>(bs[0]) | reinterpret_cast<uintptr_t>(bs[1])) & 7u);
    const bool wide_scales = (G & 3u) == 0u && __builtin_amdgcn_readfirstlane(int(scale_misalign)) == 0;
    uint2 scales_cur[2] = {make_uint2(0u, 0u), make_uint2(0u, 0u)}, scales_nxt[2] = {make_uint2(0u, 0u), make_uint2(0u, 0u)};
    // the codes of one group (8-bit) or two (4-bit, where the registers allow it) are on their way while a group is multiplied
    constexpr uint32_t kAhead = BITS == 4 ? 2u : 1u;
    BRegs<BITS> cur[2], nxt[2], nx2[2];
    const uint32_t chunks = (K + kChunkK - 1u) / kChunkK;

    // One group of 64 k: the codes of the group kAhead further on are put in flight, this group's are unpacked and
    // multiplied, and the products are scaled into the totals.
    auto group_step = [&](uint32_t c, uint32_t buf, uint32_t gi, auto wide_tag) {
        constexpr bool WIDE = decltype(wide_tag)::value;
        const uint32_t gn = min(kGroupsPerChunk * c + gi + kAhead, G - 1u);
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) load_b<BITS>(kAhead == 2u ? nx2[nt] : nxt[nt], bw[nt], WIDE ? nullptr : bs[nt], gn, kb);
        half8 af[MT][4];
#pragma unroll
        for (uint32_t mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int s = 0; s < 4; ++s)
                af[mt][s] = *reinterpret_cast<const half8 *>(&s_a[buf][mt * 32u + col][gi * 64u + kb * 32u + s * 8u]);
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
            half8 bf[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) bf[s] = b_step<BITS>(cur[nt], s);
            const uint32_t pair = gi < 2u ? scales_cur[nt].x : scales_cur[nt].y;
            const uint16_t scale_bits = WIDE ? uint16_t(pair >> (16u * (gi & 1u))) : cur[nt].scale;
            const float sc = meta_f32(scale_bits, uint32_t(META)) * kTwo24;
#pragma unroll
            for (uint32_t mt = 0; mt < MT; ++mt) {
                f32x16 p = {0};
#pragma unroll
                for (int s = 0; s < 4; ++s) p = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[mt][s], bf[s], p, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 16; ++i) total[nt][mt][i] = fmaf(sc, p[i], total[nt][mt][i]);
            }
        }
        cur[0] = nxt[0];
        cur[1] = nxt[1];
        if (kAhead == 2u) {
            nxt[0] = nx2[0];
            nxt[1] = nx2[1];
        }
    };
    auto main_loop = [&](auto wide_tag) {
        constexpr bool WIDE = decltype(wide_tag)::value;
        if (active) {
#pragma unroll
            for (int nt = 0; nt < 2; ++nt) {
                load_b<BITS>(cur[nt], bw[nt], WIDE ? nullptr : bs[nt], 0, kb);
                if (kAhead == 2u) load_b<BITS>(nxt[nt], bw[nt], WIDE ? nullptr : bs[nt], min(1u, G - 1u), kb);
                if (WIDE) scales_cur[nt] = *reinterpret_cast<const uint2 *>(bs[nt]);
            }
        }
        fetch(0);
        commit(0);
        __syncthreads();
        for (uint32_t c = 0; c < chunks; ++c) {
            const uint32_t buf = c & 1u;
            if (c + 1u < chunks) fetch(c + 1u);
            if (active) {
                if (WIDE) {  // G is a multiple of 4: every chunk is whole and its four groups are one block of code
                    if (c + 1u < chunks) {
                        scales_nxt[0] = reinterpret_cast<const uint2 *>(bs[0])[c + 1u];
                        scales_nxt[1] = reinterpret_cast<const uint2 *>(bs[1])[c + 1u];
                    }
#pragma unroll
                    for (uint32_t gi = 0; gi < kGroupsPerChunk; ++gi) group_step(c, buf, gi, wide_tag);
                    scales_cur[0] = scales_nxt[0];
                    scales_cur[1] = scales_nxt[1];
                } else {
                    const uint32_t groups_here = min(kGroupsPerChunk, G - kGroupsPerChunk * c);
                    for (uint32_t gi = 0; gi < groups_here; ++gi) group_step(c, buf, gi, wide_tag);
                }
            }
            if (c + 1u < chunks) commit(buf ^ 1u);
            __syncthreads();
        }
    };
    if (wide_scales) main_loop(std::true_type{});
    else main_loop(std::false_type{});
    // (no wave leaves here: the epilogue's barrier needs them all)

    // ---- bias term: (group sums of the rows) x (group biases), sixteen k' = eight groups an MFMA.
    // The operands of four steps are fetched together, four values a load where the rows allow it.
    if (active) {
        // a lane's four groups are one aligned 8- or 16-byte run when G is a multiple of 4 and the bias rows start aligned
        const bool wide = (G & 3u) == 0u && ((reinterpret_cast<uintptr_t>(bb[0]) | reinterpret_cast<uintptr_t>(bb[1])) & 7u) == 0u;
        for (uint32_t gbase = 0; gbase < G; gbase += 32u) {
            Frag bfr[4][2], afr[4][MT];
#pragma unroll
            for (uint32_t step = 0; step < 4; ++step) {
                const uint32_t gl = gbase + 8u * step + 4u * kb;  // this lane's four groups
                if (wide) {
                    const bool on = gl < G;
#pragma unroll
                    for (int nt = 0; nt < 2; ++nt) {
                        const uint2 b4 = on ? *reinterpret_cast<const uint2 *>(bb[nt] + gl) : make_uint2(0u, 0u);
                        bfr[step][nt].u[0] = b4.x & 0xffffu; bfr[step][nt].u[1] = b4.x >> 16;
                        bfr[step][nt].u[2] = b4.y & 0xffffu; bfr[step][nt].u[3] = b4.y >> 16;
                    }
#pragma unroll
                    for (uint32_t mt = 0; mt < MT; ++mt)
                        afr[step][mt].v = on ? *reinterpret_cast<const uint4 *>(sum_row[mt] + gl) : zero4();
                } else {
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj) {
                        const bool on = gl + jj < G;
#pragma unroll
                        for (int nt = 0; nt < 2; ++nt) bfr[step][nt].u[jj] = on ? bb[nt][gl + jj] : 0u;
#pragma unroll
                        for (uint32_t mt = 0; mt < MT; ++mt) afr[step][mt].u[jj] = on ? sum_row[mt][gl + jj] : 0u;
                    }
                }
            }
#pragma unroll
            for (uint32_t step = 0; step < 4; ++step) {
                if (gbase + 8u * step >= G) break;
#pragma unroll
                for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj) {  // the bias as fp16, doubled against (hi, lo)
                        uint16_t bits = uint16_t(bfr[step][nt].u[jj]);
                        if (META == SHRIKE_META_BF16) bits = f32_to_f16(bf16_to_f32(bits));
                        bfr[step][nt].u[jj] = uint32_t(bits) * 0x00010001u;
                    }
#pragma unroll
                    for (uint32_t mt = 0; mt < MT; ++mt)
                            total[nt][mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[step][mt].h, bfr[step][nt].h, total[nt][mt], 0, 0, 0);
                }
            }
        }
    }
    // ---- epilogue: lane holds (m = 32 mt + 8 (i / 4) + 4 kb + i % 4, n = n0 + col)
    const uint32_t n = n0 + col;
    if (MODE == 0) {
        // the main loop ended on a barrier: nobody reads the staged rows any more, and the first buffer takes the
        // tile's fp16 activations, [row][column of this block of 128]
        if (active) {
            float gab = 0.0f, uab = 0.0f;
            if (!DENSE && a.ebias) {  // moe.metal:261-269
                gab = bf16_to_f32(reinterpret_cast<const uint16_t *>(base + a.off.gate_ab_off)[n]);
                uab = bf16_to_f32(reinterpret_cast<const uint16_t *>(base + a.off.up_ab_off)[n]);
            }
#pragma unroll
            for (uint32_t mt = 0; mt < MT; ++mt) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const uint32_t m = mt * 32u + 8u * (i / 4) + 4u * kb + (i % 4);
                    float g = total[0][mt][i] + gab, u = total[1][mt][i] + uab;
                    if (DENSE && a.round_gate_up) {
                        g = f16_to_f32(f32_to_f16(g));
                        u = f16_to_f32(f32_to_f16(u));
                    }
                    s_a[0][m][wave * 32u + col] = f32_to_f16(glu_rt_fast(g, u, a.act_kind));
                }
            }
        }
        __syncthreads();
        const uint32_t c0 = col_block * 128u, columns = min(128u, N - c0);  // N is a multiple of 64
        for (uint32_t idx = threadIdx.x; idx < tile.rows * 16u; idx += 256u) {
            const uint32_t m = idx >> 4, pc = idx & 15u;
            if (pc * 8u < columns)
                *reinterpret_cast<uint4 *>(a.act + (size_t(tile_index) * kRowTile + m) * a.f + c0 + pc * 8u) =
                    *reinterpret_cast<const uint4 *>(&s_a[0][m][pc * 8u]);
        }
        uint32_t *sums_out = const_cast<uint32_t *>(a.act_sums);
        for (uint32_t slot = threadIdx.x; slot < kRowTile * 16u; slot += 256u) {  // (row, group of the block, eighth)
            const uint32_t m = slot >> 4, gl = (slot >> 3) & 1u, eighth = slot & 7u;
            const uint4 v = *reinterpret_cast<const uint4 *>(&s_a[0][m][gl * 64u + eighth * 8u]);
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
            float sum = 0.0f;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                sum = __fadd_rn(sum, f16_to_f32(uint16_t(w[t])));
                sum = __fadd_rn(sum, f16_to_f32(uint16_t(w[t] >> 16)));
            }
            sum = __fadd_rn(sum, __shfl_xor(sum, 1));
            sum = __fadd_rn(sum, __shfl_xor(sum, 2));
            sum = __fadd_rn(sum, __shfl_xor(sum, 4));
            if (eighth == 0u && m < tile.rows && gl * 64u < columns)
                sums_out[(size_t(tile_index) * kRowTile + m) * (a.f / kGroup) + c0 / kGroup + gl] = split_hi_lo(sum);
        }
    } else {
        // the down product's rows leave through the first staging buffer too, [row][column of this block of 256], and go
        // to their (token, rank) rows as whole 16-byte pieces; a call over a range of the sorted pairs writes the rows of
        // its pairs only
        const uint32_t row_lo = DENSE ? 0u : max(a.pair_lo, tile.pair_start) - tile.pair_start;
        const uint32_t row_hi = DENSE ? tile.rows : min(a.pair_hi, tile.pair_start + tile.rows) - tile.pair_start;
        if (active) {
            float dab[2] = {0.0f, 0.0f};
            if (!DENSE && a.ebias) {
                dab[0] = bf16_to_f32(reinterpret_cast<const uint16_t *>(base + a.off.down_ab_off)[n]);
                dab[1] = bf16_to_f32(reinterpret_cast<const uint16_t *>(base + a.off.down_ab_off)[n + 32u]);
            }
#pragma unroll
            for (uint32_t mt = 0; mt < MT; ++mt) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const uint32_t m = mt * 32u + 8u * (i / 4) + 4u * kb + (i % 4);
                    uint16_t y0 = f32_to_f16(total[0][mt][i] + dab[0]), y1 = f32_to_f16(total[1][mt][i] + dab[1]);
                    if (DENSE && a.scalar_gate && m < tile.rows) {  // one gate a token row (moe.metal:1195-1207)
                        const float gate_mul = 1.0f + expf(-f16_to_f32(a.scalar_gate[tile.pair_start + m]));
                        y0 = f32_to_f16(f16_to_f32(y0) / gate_mul);
                        y1 = f32_to_f16(f16_to_f32(y1) / gate_mul);
                    }
                    s_a[0][m][wave * 64u + col] = y0;
                    s_a[0][m][wave * 64u + col + 32u] = y1;
                }
            }
        }
        __syncthreads();
        const uint32_t c0 = col_block * 256u, columns = min(256u, N - c0);  // N is a multiple of 64
        constexpr uint32_t kPasses = MT * 32u * 32u / 256u;  // 32 pieces a row, 256 threads
        const uint16_t *dst_row[kPasses];
        const uint32_t pc = threadIdx.x & 31u;
#pragma unroll
        for (uint32_t pass = 0; pass < kPasses; ++pass) {
            const uint32_t m = pass * 8u + (threadIdx.x >> 5);
            const uint32_t mm = min(m, tile.rows - 1u);
            if (DENSE) {
                dst_row[pass] = a.partials + size_t(tile.pair_start + mm) * a.d;
            } else {
                const shrike_token_expert_pair p = a.pairs[tile.pair_start + mm];
                dst_row[pass] = a.partials + (size_t(p.token) * a.top_k + p.rank) * a.d;
            }
        }
#pragma unroll
        for (uint32_t pass = 0; pass < kPasses; ++pass) {
            const uint32_t m = pass * 8u + (threadIdx.x >> 5);
            if (m >= row_lo && m < row_hi && pc * 8u < columns)
                *reinterpret_cast<uint4 *>(const_cast<uint16_t *>(dst_row[pass]) + c0 + pc * 8u) = *reinterpret_cast<const uint4 *>(&s_a[0][m][pc * 8u]);
        }
    }
}

template <int BITS, int MODE, bool DENSE, int META>
__global__ __launch_bounds__(256, 2) void k_grouped_ffn(FfnArgs a) {
    warm_kernel_arguments(a);
    __shared__ __align__(16) uint16_t s_a[2][kRowTile][kLdsRow];
    // Which (row tile, column block) this workgroup takes. Workgroups go to the chip's eight XCDs (each
    // with an L2 of its own) round robin in launch order, so workgroup w runs on XCD w % 8 as that XCD's
    // item w / 8. An expert's row tiles are neighbours in the tile table: an XCD takes a contiguous run
    // of tiles with all their column blocks, so that the column blocks of a tile find its gathered rows,
    // and the row tiles of an expert its codes, in the L2 that fetched them first.
    const uint32_t column_blocks = gridDim.y;
    const uint32_t tile_total = DENSE ? (a.dense_rows + kRowTile - 1u) / kRowTile : *a.tile_count;
    const uint32_t w = blockIdx.y * gridDim.x + blockIdx.x;
    const uint32_t xcd = w & 7u, item = w >> 3;
    // tiles an XCD takes: an eighth of them, the first (total mod 8) XCDs one more
    const uint32_t run = tile_total / 8u + (xcd < tile_total % 8u ? 1u : 0u), first = xcd * (tile_total / 8u) + min(xcd, tile_total % 8u);
    const uint32_t place = item / column_blocks, col_block = item % column_blocks;  // the workgroup's place in its XCD's run
    if (place >= run) return;
    uint32_t tile_index = first + place;
    shrike_row_tile tile;
    if (DENSE) {
        if (tile_index >= tile_total) return;
        tile.cell = 0;
        tile.pair_start = tile_index * kRowTile;
        tile.rows = min(kRowTile, a.dense_rows - tile.pair_start);
        tile.expert = 0;
    } else {
        if (tile_index >= tile_total) return;
        // Which tile of the table the workgroup takes. A compute unit holds two of these workgroups, whose waves share its
        // SIMDs' issue, and an XCD's workgroups reach its compute units in launch order, one each before any gets a second
        // (read from the hardware: item i and item i + 32 of an XCD share a unit). A tile of more than 32 rows is twice a
        // smaller one's matrix work, and the launch ends with the units that hold two of those.
        //  - Where the gate/up launch fits the chip at once: every XCD takes the same number of the larger tiles (a block of
        //    them in table order, so an expert's stay together) and fills its eighth with a block of the smaller ones; the
        //    larger go first, so each gets a smaller neighbour.
        //  - Otherwise the XCD's eighth is a contiguous run of the table, its larger tiles first: the workgroups that start
        //    late are then the short ones, on the XCDs with the least work.
        // A lane reads one record; the chosen one is read across (no second load).
        const uint32_t lane = threadIdx.x & 63u;
        const uint32_t gate_up_blocks = (a.f + 127u) / 128u;
        bool chosen = false;
        if (tile_total <= 256u && tile_total * gate_up_blocks <= a.resident_workgroups) {
            // (four named records, not an array: the compiler kept an array of them in private memory)
            const uint4 *table = reinterpret_cast<const uint4 *>(a.tiles);
            const uint4 rec0 = lane < tile_total ? table[lane] : zero4();
            const uint4 rec1 = lane + 64u < tile_total ? table[lane + 64u] : zero4();
            const uint4 rec2 = lane + 128u < tile_total ? table[lane + 128u] : zero4();
            const uint4 rec3 = lane + 192u < tile_total ? table[lane + 192u] : zero4();
            const bool in0 = lane < tile_total, in1 = lane + 64u < tile_total, in2 = lane + 128u < tile_total, in3 = lane + 192u < tile_total;
            const uint64_t larger0 = __ballot(in0 && rec0.z > 32u), larger1 = __ballot(in1 && rec1.z > 32u);
            const uint64_t larger2 = __ballot(in2 && rec2.z > 32u), larger3 = __ballot(in3 && rec3.z > 32u);
            const uint64_t smaller0 = __ballot(in0 && rec0.z <= 32u), smaller1 = __ballot(in1 && rec1.z <= 32u);
            const uint64_t smaller2 = __ballot(in2 && rec2.z <= 32u), smaller3 = __ballot(in3 && rec3.z <= 32u);
            const uint32_t larger_total = uint32_t(__popcll(larger0) + __popcll(larger1) + __popcll(larger2) + __popcll(larger3));
            const uint32_t lq = larger_total / 8u, lr = larger_total % 8u;
            if (lq + 1u <= tile_total / 8u) {  // every XCD's share of the larger tiles fits its eighth
                const uint32_t mine_larger = lq + (xcd < lr ? 1u : 0u), larger_first = xcd * lq + min(xcd, lr);
                const bool take_larger = place < mine_larger;
                uint32_t want = take_larger ? larger_first + place : (first - larger_first) + (place - mine_larger);
                const uint64_t m0 = take_larger ? larger0 : smaller0, m1 = take_larger ? larger1 : smaller1;
                const uint64_t m2 = take_larger ? larger2 : smaller2, m3 = take_larger ? larger3 : smaller3;
                const uint32_t c0 = uint32_t(__popcll(m0)), c1 = uint32_t(__popcll(m1)), c2 = uint32_t(__popcll(m2));
                uint64_t set;
                uint32_t block;
                if (want < c0) { set = m0; block = 0; }
                else if (want < c0 + c1) { set = m1; block = 1; want -= c0; }
                else if (want < c0 + c1 + c2) { set = m2; block = 2; want -= c0 + c1; }
                else { set = m3; block = 3; want -= c0 + c1 + c2; }
                chosen = want < uint32_t(__popcll(set));
                if (chosen) {
                    const bool me = ((set >> lane) & 1ull) != 0ull && uint32_t(__popcll(set & ((1ull << lane) - 1ull))) == want;
                    const int src = __builtin_amdgcn_readfirstlane(__ffsll((long long)__ballot(me)) - 1);
                    auto take = [&](const uint4 &r) {  // (a branch a block, uniform: a select between the four records became an
                                                       // indexed load from private memory)
                        tile.cell = uint32_t(__builtin_amdgcn_readlane(int(r.x), src));
                        tile.pair_start = uint32_t(__builtin_amdgcn_readlane(int(r.y), src));
                        tile.rows = uint32_t(__builtin_amdgcn_readlane(int(r.z), src));
                        tile.expert = uint32_t(__builtin_amdgcn_readlane(int(r.w), src));
                    };
                    if (block == 0) take(rec0);
                    else if (block == 1) take(rec1);
                    else if (block == 2) take(rec2);
                    else take(rec3);
                    tile_index = 64u * block + uint32_t(src);
                }
            }
        }
        const uint32_t count = run;
        if (chosen) {
        } else if (count <= 64u) {
            const uint4 rec = lane < count ? reinterpret_cast<const uint4 *>(a.tiles)[first + lane] : zero4();
            const uint64_t heavy = __ballot(lane < count && rec.z > 32u), light = __ballot(lane < count && rec.z <= 32u);
            const uint32_t heavies = uint32_t(__popcll(heavy));
            const uint64_t set = place < heavies ? heavy : light;
            const uint32_t want = place < heavies ? place : place - heavies;
            const bool mine = ((set >> lane) & 1ull) != 0ull && uint32_t(__popcll(set & ((1ull << lane) - 1ull))) == want;
            const int src = __builtin_amdgcn_readfirstlane(__ffsll((long long)__ballot(mine)) - 1);
            tile.cell = uint32_t(__builtin_amdgcn_readlane(int(rec.x), src));
            tile.pair_start = uint32_t(__builtin_amdgcn_readlane(int(rec.y), src));
            tile.rows = uint32_t(__builtin_amdgcn_readlane(int(rec.z), src));
            tile.expert = uint32_t(__builtin_amdgcn_readlane(int(rec.w), src));
            tile_index = first + uint32_t(src);
        } else {
            tile = a.tiles[tile_index];
        }
        if (a.residency) {  // moe.metal:136-146: a hit names its cell, anything else is the sentinel
            const uint64_t word = a.residency[tile.expert];
            tile.cell = uint32_t(word >> 32) == SHRIKE_RESIDENCY_RESIDENT ? uint32_t(word) : kSentinel;
        }
        if (tile.cell == kSentinel || tile.rows == 0) return;
        if (tile.pair_start + tile.rows <= a.pair_lo || tile.pair_start >= a.pair_hi) return;
    }

    if (tile.rows > 32u) ffn_tile<BITS, MODE, DENSE, 2, META>(a, tile, tile_index, col_block, s_a);
    else ffn_tile<BITS, MODE, DENSE, 1, META>(a, tile, tile_index, col_block, s_a);
}

int launch_row_group_sums(const uint16_t *src, size_t stride, uint32_t rows, uint32_t n, uint32_t *out,
                          const uint32_t *row_limit_tiles, hipStream_t s);

template <int BITS, bool DENSE, int META>
static int launch_ffn_meta(const FfnArgs &a, uint32_t max_tiles, hipStream_t s) {
    const dim3 block(256);
    const uint32_t grid_tiles = (max_tiles + 7u) & ~7u;  // whole runs for the kernel's XCD mapping
    hipLaunchKernelGGL((k_grouped_ffn<BITS, 0, DENSE, META>), dim3(grid_tiles, (a.f + 127u) / 128u), block, 0, s, a);
    SHRIKE_HIP(hipGetLastError());
    // (the activations' group sums were written by the gate/up launch itself)
    hipLaunchKernelGGL((k_grouped_ffn<BITS, 1, DENSE, META>), dim3(grid_tiles, (a.d + 255u) / 256u), block, 0, s, a);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}
template <int BITS, bool DENSE>
static int launch_ffn(const FfnArgs &a, uint32_t max_tiles, hipStream_t s) {
    return a.meta == SHRIKE_META_F16 ? launch_ffn_meta<BITS, DENSE, SHRIKE_META_F16>(a, max_tiles, s)
                                     : launch_ffn_meta<BITS, DENSE, SHRIKE_META_BF16>(a, max_tiles, s);
}

// Two workgroups of the FFN kernels a compute unit (their registers and LDS allow no more).
static uint32_t resident_ffn_workgroups() {
    int device = 0, units = 0;
    if (hipGetDevice(&device) != hipSuccess || hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess)
        return 0;
    return 2u * uint32_t(units);
}

struct Workspace {
    size_t hidden_sums, act, act_sums, total;
};
static Workspace workspace_layout(uint32_t query_count, uint32_t max_tiles, uint32_t d, uint32_t f) {
    auto round = [](size_t v) { return (v + 255u) & ~size_t(255); };
    Workspace w;
    w.hidden_sums = 0;
    w.act = round(size_t(query_count) * (d / kGroup) * 4u);
    w.act_sums = w.act + round(size_t(max_tiles) * kRowTile * f * 2u);
    w.total = w.act_sums + round(size_t(max_tiles) * kRowTile * (f / kGroup) * 4u);
    return w;
}

}  // namespace shrike

using namespace shrike;

extern "C" {
size_t shrike_hip_prefill_ffn_workspace_bytes(uint32_t query_count, uint32_t max_row_tiles, uint32_t d, uint32_t f) {
    return workspace_layout(query_count, max_row_tiles, d, f).total;
}

static int grouped_ffn(shrike_hip_moe *moe, void *stream, const shrike_pool_bases *pool, uint64_t pool_slot_stride,
                       const shrike_expert_offsets *offsets, const shrike_hip_grouped_routes *routes, uint32_t max_row_tiles,
                       const uint64_t *d_residency, uint32_t pair_lo, uint32_t pair_hi, const void *d_hidden,
                       uint32_t hidden_stride_elements, void *d_route_partials, void *d_workspace, size_t workspace_bytes,
                       uint32_t query_count, uint32_t d, uint32_t f, uint32_t top_k, bool presummed = false) {
    SHRIKE_REQUIRE(moe && pool && offsets && routes, "grouped FFN: NULL argument");
    SHRIKE_REQUIRE(d == moe->desc.d && f == moe->desc.f, "grouped FFN: shape %ux%u differs from the handle's %ux%u", d, f, moe->desc.d, moe->desc.f);
    SHRIKE_REQUIRE(d % kGroup == 0 && f % kGroup == 0 && d > 0 && f > 0, "D and F must be positive multiples of 64");
    SHRIKE_REQUIRE(top_k > 0, "topK must be positive");
    SHRIKE_REQUIRE(hidden_stride_elements >= d && hidden_stride_elements % 8u == 0, "hidden stride is too small or leaves rows unaligned");
    SHRIKE_REQUIRE(routes->sorted_pairs && routes->row_tiles && routes->row_tile_count, "grouped FFN: routes are not bound");
    SHRIKE_REQUIRE(d_hidden && d_route_partials && d_workspace, "grouped FFN: NULL buffer");
    SHRIKE_REQUIRE(reinterpret_cast<uintptr_t>(d_workspace) % 256u == 0, "grouped FFN: workspace must be 256-byte aligned");
    SHRIKE_REQUIRE(pool->cells_per_chunk > 0 && pool_slot_stride % 16u == 0, "grouped FFN: bad pool geometry");
    if (int rc = check_offsets(offsets, d, f, moe->desc.routed_weight_bits)) return rc;
    if (max_row_tiles == 0 || query_count == 0 || pair_lo >= pair_hi) return 0;
    const Workspace w = workspace_layout(query_count, max_row_tiles, d, f);
    SHRIKE_REQUIRE(workspace_bytes >= w.total, "grouped FFN: workspace of %zu bytes, %zu needed", workspace_bytes, w.total);
    uint8_t *ws = static_cast<uint8_t *>(d_workspace);
    FfnArgs a = {};
    fill_pool(a.pool, pool);
    a.stride = pool_slot_stride;
    a.off = *offsets;
    a.tiles = routes->row_tiles;
    a.tile_count = routes->row_tile_count;
    a.residency = d_residency;
    a.pair_lo = pair_lo;
    a.pair_hi = pair_hi;
    a.pairs = static_cast<const shrike_token_expert_pair *>(routes->sorted_pairs);
    a.hidden = static_cast<const uint16_t *>(d_hidden);
    a.hidden_stride = hidden_stride_elements;
    a.hidden_sums = reinterpret_cast<uint32_t *>(ws + w.hidden_sums);
    a.act = reinterpret_cast<uint16_t *>(ws + w.act);
    a.act_sums = reinterpret_cast<uint32_t *>(ws + w.act_sums);
    a.partials = static_cast<uint16_t *>(d_route_partials);
    a.d = d; a.f = f; a.top_k = top_k;
    a.meta = moe->desc.meta_dtype;
    a.act_kind = moe->desc.activation;
    a.ebias = moe->desc.expert_additive_biases;
    a.resident_workgroups = resident_ffn_workgroups();
    hipStream_t s = as_stream(stream);
    if (!presummed)
        if (int rc = launch_row_group_sums(a.hidden, hidden_stride_elements, query_count, d, const_cast<uint32_t *>(a.hidden_sums), nullptr, s)) return rc;
    return moe->desc.routed_weight_bits == 8 ? launch_ffn<8, false>(a, max_row_tiles, s) : launch_ffn<4, false>(a, max_row_tiles, s);
}

int shrike_hip_prefill_grouped_ffn(shrike_hip_moe *moe, void *stream, const shrike_pool_bases *pool,
                                   uint64_t pool_slot_stride, const shrike_expert_offsets *offsets,
                                   const shrike_hip_grouped_routes *routes, uint32_t max_row_tiles, const void *d_hidden,
                                   uint32_t hidden_stride_elements, void *d_route_partials, void *d_workspace,
                                   size_t workspace_bytes, uint32_t query_count, uint32_t d, uint32_t f, uint32_t top_k) {
    return grouped_ffn(moe, stream, pool, pool_slot_stride, offsets, routes, max_row_tiles, nullptr, 0u, 0xffffffffu, d_hidden,
                       hidden_stride_elements, d_route_partials, d_workspace, workspace_bytes, query_count, d, f, top_k);
}

int shrike_hip_prefill_grouped_ffn_presummed(shrike_hip_moe *moe, void *stream, const shrike_pool_bases *pool,
                                             uint64_t pool_slot_stride, const shrike_expert_offsets *offsets,
                                             const shrike_hip_grouped_routes *routes, uint32_t max_row_tiles,
                                             const void *d_hidden, uint32_t hidden_stride_elements, void *d_route_partials,
                                             void *d_workspace, size_t workspace_bytes, uint32_t query_count, uint32_t d,
                                             uint32_t f, uint32_t top_k) {
    return grouped_ffn(moe, stream, pool, pool_slot_stride, offsets, routes, max_row_tiles, nullptr, 0u, 0xffffffffu, d_hidden,
                       hidden_stride_elements, d_route_partials, d_workspace, workspace_bytes, query_count, d, f, top_k, true);
}

int shrike_hip_prefill_streamed_batched(shrike_hip_moe *moe, void *stream, const shrike_pool_bases *pool,
                                        uint64_t pool_slot_stride, const shrike_expert_offsets *offsets,
                                        const shrike_hip_grouped_routes *routes, uint32_t max_row_tiles,
                                        const uint64_t *d_residency, uint32_t pair_start, uint32_t pair_count,
                                        uint32_t pair_microbatch_rows, const void *d_hidden, uint32_t hidden_stride_elements,
                                        void *d_route_partials, void *d_workspace, size_t workspace_bytes,
                                        uint32_t query_count, uint32_t d, uint32_t f, uint32_t top_k,
                                        uint32_t *out_microbatches) {
    if (out_microbatches) *out_microbatches = 0;
    // PrefillGroupedRoutedMoE.swift:861-863: nothing to do is not an error
    if (pair_count == 0 || pair_microbatch_rows == 0) return 0;
    SHRIKE_REQUIRE(uint64_t(pair_start) + pair_count <= uint64_t(query_count) * top_k, "streamed batch: pairs %u..%llu leave the chunk's %llu",
                   pair_start, (unsigned long long)pair_start + pair_count, (unsigned long long)query_count * top_k);
    if (int rc = grouped_ffn(moe, stream, pool, pool_slot_stride, offsets, routes, max_row_tiles, d_residency, pair_start,
                             pair_start + pair_count, d_hidden, hidden_stride_elements, d_route_partials, d_workspace,
                             workspace_bytes, query_count, d, f, top_k))
        return rc;
    if (out_microbatches) *out_microbatches = (pair_count + pair_microbatch_rows - 1u) / pair_microbatch_rows;
    return 0;
}

size_t shrike_hip_prefill_shared_expert_workspace_bytes(uint32_t query_count, uint32_t d, uint32_t f_shared) {
    return workspace_layout(query_count, (query_count + kRowTile - 1u) / kRowTile, d, f_shared).total;
}

int shrike_hip_prefill_shared_expert(shrike_hip_moe *moe, void *stream, const shrike_projection *gate,
                                     const shrike_projection *up, const shrike_projection *down, uint32_t bits,
                                     const void *d_hidden, uint32_t hidden_stride_elements, void *d_h1, const void *d_scalar_gate,
                                     void *d_workspace, size_t workspace_bytes, uint32_t query_count, uint32_t d,
                                     uint32_t f_shared) {
    SHRIKE_REQUIRE(moe != nullptr, "moe handle is NULL");
    if (int rc = check_shared(gate, up, down, bits, d, f_shared)) return rc;
    SHRIKE_REQUIRE(hidden_stride_elements >= d && hidden_stride_elements % 8u == 0, "hidden stride is too small or leaves rows unaligned");
    SHRIKE_REQUIRE(d_hidden && d_h1 && d_workspace, "shared expert: NULL buffer");
    SHRIKE_REQUIRE(reinterpret_cast<uintptr_t>(d_workspace) % 256u == 0, "shared expert: workspace must be 256-byte aligned");
    if (query_count == 0) return 0;
    const uint32_t tiles = (query_count + kRowTile - 1u) / kRowTile;
    const Workspace w = workspace_layout(query_count, tiles, d, f_shared);
    SHRIKE_REQUIRE(workspace_bytes >= w.total, "shared expert: workspace of %zu bytes, %zu needed", workspace_bytes, w.total);
    uint8_t *ws = static_cast<uint8_t *>(d_workspace);
    FfnArgs a = {};
    a.hidden = static_cast<const uint16_t *>(d_hidden);
    a.hidden_stride = hidden_stride_elements;
    a.hidden_sums = reinterpret_cast<uint32_t *>(ws + w.hidden_sums);
    a.act = reinterpret_cast<uint16_t *>(ws + w.act);
    a.act_sums = reinterpret_cast<uint32_t *>(ws + w.act_sums);
    a.partials = static_cast<uint16_t *>(d_h1);
    a.d = d; a.f = f_shared; a.top_k = 1;
    a.meta = moe->desc.meta_dtype;
    a.act_kind = moe->desc.activation;
    const shrike_projection *proj[3] = {gate, up, down};
    for (int i = 0; i < 3; ++i) {
        a.dense_w[i] = static_cast<const uint8_t *>(proj[i]->weights);
        a.dense_s[i] = static_cast<const uint16_t *>(proj[i]->scales);
        a.dense_b[i] = static_cast<const uint16_t *>(proj[i]->biases);
    }
    a.dense_rows = query_count;
    a.round_gate_up = 1;
    a.scalar_gate = static_cast<const uint16_t *>(d_scalar_gate);
    hipStream_t s = as_stream(stream);
    if (int rc = launch_row_group_sums(a.hidden, hidden_stride_elements, query_count, d, const_cast<uint32_t *>(a.hidden_sums), nullptr, s)) return rc;
    return bits == 8 ? launch_ffn<8, true>(a, tiles, s) : launch_ffn<4, true>(a, tiles, s);
}

}  // extern "C"
