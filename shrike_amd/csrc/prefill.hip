// The prefill side of the routed path for gfx950, except the grouped FFN: the router for a
// block of tokens, the token->expert grouping as a stable counting sort, the per-row group
// sums the grouped FFN folds the affine biases with, the token-major reduce and the
// residual add.
#include "prefill_common.h"
#include "router_row.h"

#include "../../include/shrike_host.h"

namespace shrike {

constexpr uint32_t kRouterTokenBlock = 4;  // tokens a wave runs one expert row against

// prefill.metal:369-439: logits of every (token, expert). A wave holds one expert and walks
// kRouterTokenBlock tokens, so the row comes from HBM once and from L1 afterwards. The row
// arithmetic is the decode router's, operand for operand.
template <int RK>
__global__ __launch_bounds__(256) void k_prefill_logits(RouterArgs a, uint32_t query_count, uint32_t stride, float *ws) {
    warm_kernel_arguments(a);
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t e = blockIdx.x * 4u + wave;
    if (e >= a.sel.num_experts) return;
#pragma unroll 1
    for (uint32_t i = 0; i < kRouterTokenBlock; ++i) {
        const uint32_t t = blockIdx.y * kRouterTokenBlock + i;
        if (t >= query_count) break;
        RouterArgs b = a;
        b.hidden = a.hidden + size_t(t) * stride;
        b.logits_out = ws + size_t(t) * a.sel.num_experts;
        router_row<RK>(b, e, lane);
    }
}

// The fp16 router's fast path. x * effective_scale is the same for every expert: a workgroup forms
// the products (router_row's, moe.metal:357-358) once per token while staging the row in LDS, keeps its
// experts' rows in registers and walks a block of tokens, the next step's rows in flight while one is
// multiplied. The additions are router_row's, in router_row's order, so the logits are the same bits.

// A wave keeps ROWS fp16 router rows in registers (MAXI 16-byte chunks a lane and row); the workgroup
// walks a block of TOKENS tokens, TPS of them a step: their x rows are staged once in LDS (the next
// step's in flight while one is multiplied) for the four waves to read, and the TPS * ROWS sums of a step
// go through the butterfly side by side. Every logit is summed in the decode router's order (lane l:
// chunks l, l+64, ..., xor butterfly).
// One stage of the split butterfly over LIVE sums (a power of two above 1) at lane distance 32 >> STAGE: the partner with
// the distance's bit set keeps the upper half of the sums and sends the lower, the other the reverse; each adds the
// partner's copy of what it keeps. LIVE / 2 sums are left in v[0 .. LIVE / 2).
template <uint32_t LIVE, uint32_t STAGE>
__device__ __forceinline__ void split_stage(float *v, uint32_t lane) {
    constexpr int kDistance = 32 >> STAGE;
    const bool upper = (lane & uint32_t(kDistance)) != 0u;
#pragma unroll
    for (uint32_t j = 0; j < LIVE / 2u; ++j) {
        const float keep = upper ? v[j + LIVE / 2u] : v[j], send = upper ? v[j] : v[j + LIVE / 2u];
        v[j] = __fadd_rn(keep, __shfl_xor(send, kDistance));
    }
}
template <uint32_t SUMS, uint32_t STAGES>
__device__ __forceinline__ void split_stages(float *v, uint32_t lane) {
    if constexpr (STAGES >= 1u) split_stage<SUMS, 0>(v, lane);
    if constexpr (STAGES >= 2u) split_stage<SUMS / 2u, 1>(v, lane);
    if constexpr (STAGES >= 3u) split_stage<SUMS / 4u, 2>(v, lane);
}

template <int MAXI, int ROWS, uint32_t TOKENS, uint32_t TPS>
__global__ __launch_bounds__(256) void k_prefill_logits_f16(const uint16_t *weights, const uint16_t *hidden, uint32_t stride,
                                                            const uint16_t *eff, float *logits, uint32_t query_count,
                                                            uint32_t num_experts, uint32_t d) {
    // chunk c = lane + 64 i of a row is two float4: half h of it sits at [(2 i + h) * 64 + lane], so that a
    // wave's read of one half is one contiguous kilobyte
    __shared__ float4 s_x[2][TPS][MAXI * 2 * 64];
    const uint32_t lane = threadIdx.x & 63u, wave = wave_index();
    const uint32_t e0 = (blockIdx.x * 4u + wave) * ROWS;
    const uint32_t chunks = d / 8u;
    // the rows stay packed: a multiply-add that takes its fp16 factor as it is (v_fma_mix_f32) widens it
    // exactly, so the sums are those of converting first, and a row costs half the registers
    uint4 w[ROWS][MAXI];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const uint32_t e = min(e0 + uint32_t(r), num_experts - 1u);  // past the last row: a copy, never stored
#pragma unroll
        for (int i = 0; i < MAXI; ++i) {
            const uint32_t c = lane + 64u * i;
            w[r][i] = *reinterpret_cast<const uint4 *>(weights + size_t(e) * d + size_t(c < chunks ? c : 0u) * 8u);
        }
    }
    const uint32_t t0 = blockIdx.y * TOKENS;
    const uint32_t t1 = min(t0 + TOKENS, query_count);
    if (t0 >= t1) return;
    // a thread stages kStage 8-element chunks of a token's row: fp16 x times bf16 effective scale, the
    // exact fp32 product, two float4 a chunk
    static_assert(MAXI % 4 == 0, "a workgroup of 256 threads stages 64 * MAXI chunks a token");
    constexpr int kStage = MAXI / 4;
    uint4 eff_c[kStage];
#pragma unroll
    for (int j = 0; j < kStage; ++j) eff_c[j] = reinterpret_cast<const uint4 *>(eff)[min(threadIdx.x + 256u * j, chunks - 1u)];
    auto stage_load = [&](uint4 (&st)[TPS][kStage], uint32_t t) {
#pragma unroll
        for (uint32_t u = 0; u < TPS; ++u) {
            const uint4 *row = reinterpret_cast<const uint4 *>(hidden + size_t(min(t + u, t1 - 1u)) * stride);
#pragma unroll
            for (int j = 0; j < kStage; ++j) st[u][j] = row[min(threadIdx.x + 256u * j, chunks - 1u)];  // past the row: a copy, never stored
        }
    };
    auto stage_store = [&](const uint4 (&st)[TPS][kStage], uint32_t buf) {
#pragma unroll
        for (uint32_t u = 0; u < TPS; ++u)
#pragma unroll
            for (int j = 0; j < kStage; ++j) {
                const uint32_t c = threadIdx.x + 256u * j;
                const uint4 xv = st[u][j], ev = eff_c[j];
                const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w}, ew[4] = {ev.x, ev.y, ev.z, ev.w};
                float o[8];
#pragma unroll
                for (int q = 0; q < 4; ++q) {  // moe.metal:357-358 (exact product)
                    o[2 * q] = __fmul_rn(f16_to_f32(uint16_t(xw[q])), bf16_to_f32(uint16_t(ew[q])));
                    o[2 * q + 1] = __fmul_rn(f16_to_f32(uint16_t(xw[q] >> 16)), bf16_to_f32(uint16_t(ew[q] >> 16)));
                }
                if (c < chunks) {
                    s_x[buf][u][(2u * (c >> 6)) * 64u + (c & 63u)] = make_float4(o[0], o[1], o[2], o[3]);
                    s_x[buf][u][(2u * (c >> 6) + 1u) * 64u + (c & 63u)] = make_float4(o[4], o[5], o[6], o[7]);
                }
            }
    };
    auto step = [&](uint32_t buf, uint32_t t) {
        float acc[TPS][ROWS];
#pragma unroll
        for (uint32_t u = 0; u < TPS; ++u)
#pragma unroll
            for (int r = 0; r < ROWS; ++r) acc[u][r] = 0.0f;
#pragma unroll
        for (int i = 0; i < MAXI; ++i) {
            if (lane + 64u * i < chunks) {
                uint32_t ww[ROWS][4];
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    // the widening belongs to the multiply-add: keep it from being hoisted out of the token loop. The row's own
                    // registers are named as changed (they are not), so that nothing is copied for it.
                    asm volatile("" : "+v"(w[r][i].x), "+v"(w[r][i].y), "+v"(w[r][i].z), "+v"(w[r][i].w));
                    ww[r][0] = w[r][i].x; ww[r][1] = w[r][i].y; ww[r][2] = w[r][i].z; ww[r][3] = w[r][i].w;
                }
#pragma unroll
                for (uint32_t u = 0; u < TPS; ++u) {
                    const float4 x0 = s_x[buf][u][(2 * i) * 64 + lane], x1 = s_x[buf][u][(2 * i + 1) * 64 + lane];
                    const float xv[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
#pragma unroll
                    for (int r = 0; r < ROWS; ++r)
#pragma unroll
                        for (int j = 0; j < 8; ++j)
                            acc[u][r] = fmaf(f16_to_f32(uint16_t(ww[r][j / 2] >> (16 * (j % 2)))), xv[j], acc[u][r]);
                }
            }
        }
        // The butterfly of router_row (xor 32, 16, ..., 1) over the step's TPS * ROWS sums at once. While more than one
        // sum is left, a step's two partner lanes split them: each keeps half and adds the partner's copy of that half,
        // so a step costs half the exchanges of the one before; what a lane adds is what the plain butterfly adds in that
        // lane (the same two operands, and addition commutes), so every sum is router_row's bit for bit. Sum j ends in the
        // lanes whose upper bits spell j.
        constexpr uint32_t kSums = TPS * uint32_t(ROWS);
        static_assert(kSums == 1u || kSums == 2u || kSums == 4u || kSums == 8u, "the split butterfly takes 1, 2, 4 or 8 sums");
        float v[kSums];
#pragma unroll
        for (uint32_t u = 0; u < TPS; ++u)
#pragma unroll
            for (int r = 0; r < ROWS; ++r) v[u * ROWS + r] = acc[u][r];
        // (every index below is a constant: with the number of live sums in a variable the compiler kept v in private memory)
        constexpr uint32_t kSplitStages = kSums == 8u ? 3u : kSums == 4u ? 2u : kSums == 2u ? 1u : 0u;
        split_stages<kSums, kSplitStages>(v, lane);
#pragma unroll
        for (int o = 32 >> kSplitStages; o >= 1; o >>= 1) v[0] = __fadd_rn(v[0], __shfl_xor(v[0], o));
        // which sum this lane holds: one bit a split, from the first split (xor 32) down
        constexpr uint32_t kSplits = kSums == 8u ? 3u : kSums == 4u ? 2u : kSums == 2u ? 1u : 0u;
        const uint32_t mine = kSplits ? lane >> (6u - kSplits) : 0u;
        if ((lane & ((64u >> kSplits) - 1u)) == 0u) {
            const uint32_t u = mine / uint32_t(ROWS), r = mine % uint32_t(ROWS);
            if (t + u < t1 && e0 + r < num_experts) logits[size_t(t + u) * num_experts + e0 + r] = v[0];
        }
    };
    uint4 staged[TPS][kStage];  // live across a step's arithmetic; handed to the lambdas as a parameter so it stays in registers
    stage_load(staged, t0);
    stage_store(staged, 0);
    __syncthreads();
    uint32_t buf = 0;
    for (uint32_t t = t0; t < t1; t += TPS, buf ^= 1u) {
        const bool more = t + TPS < t1;
        if (more) stage_load(staged, t + TPS);
        step(buf, t);
        if (more) stage_store(staged, buf ^ 1u);
        __syncthreads();
    }
}

constexpr uint32_t kLogitTokens = 8;  // tokens a workgroup walks with its rows: small blocks, many workgroups
constexpr uint32_t kLogitTokensPerStep = 2;

template <int MAXI, int ROWS>
static void launch_prefill_logits_f16(const uint16_t *weights, const uint16_t *hidden, uint32_t stride, const uint16_t *eff,
                                      float *logits, uint32_t query_count, uint32_t num_experts, uint32_t d, hipStream_t s) {
    const uint32_t per_block = 4u * ROWS;
    hipLaunchKernelGGL((k_prefill_logits_f16<MAXI, ROWS, kLogitTokens, kLogitTokensPerStep>),
                       dim3((num_experts + per_block - 1u) / per_block, (query_count + kLogitTokens - 1u) / kLogitTokens),
                       dim3(256), 0, s, weights, hidden, stride, eff, logits, query_count, num_experts, d);
}

// prefill.metal:441-563: one wave selects for one token.
// group_sums (may be null): the wave also leaves, for its token's row of `hidden`, the sum of every group of 64 of its fp16
// elements, exactly as k_row_group_sums forms it (a lane takes an 8-element chunk: its eight values in order, then eight
// neighbouring lanes fold pairwise), as (hi, lo) halves at [token][group]. The launch is a chain of dependent steps on half the
// chip's compute units: the row's loads go out ahead of the selection and are summed behind it.
template <bool SUMS>
__global__ __launch_bounds__(256) void k_prefill_select(SelectArgs sel, const float *ws, uint32_t *out_indices,
                                                        uint16_t *out_weights, uint32_t query_count, const uint16_t *hidden,
                                                        uint32_t stride, uint32_t d, uint32_t *group_sums) {
    warm_kernel_arguments(sel);
    __shared__ RouteScratch s_route[4];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t t = blockIdx.x * 4u + wave;
    if (t >= query_count) return;
    constexpr uint32_t kAhead = SHRIKE_MAX_HIDDEN / 8u / 64u;  // chunks a lane can own
    uint4 mine[SUMS ? kAhead : 1u];
    const uint32_t chunks = d / 8u;
    if (SUMS) {
        const uint4 *row = reinterpret_cast<const uint4 *>(hidden + size_t(t) * stride);
#pragma unroll
        for (uint32_t i = 0; i < kAhead; ++i)
            if (64u * i < chunks) mine[i] = row[min(lane + 64u * i, chunks - 1u)];  // past the row: a copy, never stored
    }
    sel.logits = ws + size_t(t) * sel.num_experts;
    RouteLists lists = {};
    lists.out_indices = out_indices + size_t(t) * sel.top_k;
    lists.out_weights = out_weights + size_t(t) * sel.top_k;
    uint32_t cell;
    route_wave<false>(sel, lists, lane, true, cell, s_route[wave]);
    if (SUMS) {
#pragma unroll
        for (uint32_t i = 0; i < kAhead; ++i) {
            if (64u * i >= chunks) break;
            const uint32_t c = lane + 64u * i;
            const uint32_t xw[4] = {mine[i].x, mine[i].y, mine[i].z, mine[i].w};
            float sum = 0.0f;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                sum = __fadd_rn(sum, f16_to_f32(uint16_t(xw[q])));
                sum = __fadd_rn(sum, f16_to_f32(uint16_t(xw[q] >> 16)));
            }
            sum = __fadd_rn(sum, __shfl_xor(sum, 1));
            sum = __fadd_rn(sum, __shfl_xor(sum, 2));
            sum = __fadd_rn(sum, __shfl_xor(sum, 4));
            if (c < chunks && (c & 7u) == 0u) group_sums[size_t(t) * (d / 64u) + (c >> 3)] = split_hi_lo(sum);  // d % 64 == 0: whole groups
        }
    }
}

// ---- grouping ---------------------------------------------------------------------------

struct GroupArgs {
    const uint32_t *indices;
    const uint16_t *weights;
    uint32_t pairs, top_k, num_experts;
    const uint64_t *sort_keys, *residency;
    shrike_token_expert_pair *sorted;
    uint32_t *offsets, *counts;
    shrike_row_tile *tiles;
    uint32_t *tile_count;
};

constexpr uint32_t kGroupLdsPairs = 49152;   // pairs whose expert ids (one byte each) fit the LDS copy
constexpr uint32_t kGroupLdsWeights = 16384;  // pairs whose fp16 weights are staged beside them

// One launch, four experts a workgroup (one a wave). Every workgroup builds the whole
// histogram for itself in LDS (the pairs are a few KB and sit in L2), so no count has to
// cross workgroups. A wave then knows its expert's first position (the pairs of every
// expert ordered before it), writes its row tiles, and writes its pairs in index order.
// The pairs arrive token-major, so index order is (token, rank) order: the permutation
// equals the reference's sort by (sort key, expert, token, rank)
// (PrefillMoEGrouping.swift:323-332).
__global__ __launch_bounds__(256) void k_group(GroupArgs a) {
    warm_kernel_arguments(a);
    __shared__ uint32_t s_hist[SHRIKE_MAX_ROUTER_EXPERTS];
    __shared__ __align__(16) uint8_t s_ids[kGroupLdsPairs];
    __shared__ uint16_t s_weights[kGroupLdsWeights];
    const bool in_lds = a.pairs <= kGroupLdsPairs;
    // the placement loop below is one dependent step a 64 pairs: a global load inside it would
    // cost its full latency every step
    const bool weights_in_lds = a.pairs <= kGroupLdsWeights;
    s_hist[threadIdx.x] = 0u;
    __syncthreads();
    // sixteen pairs a thread at a time: all their loads go out before the first is used (with the uses
    // inside the loading loop every load was waited for on the spot, thirty-two round trips to L2 on end)
    constexpr uint32_t kPairsAThread = 16;
    for (uint32_t base = 0; base < a.pairs; base += 256u * kPairsAThread) {
        uint32_t v[kPairsAThread];
        uint16_t wv[kPairsAThread];
#pragma unroll
        for (uint32_t j = 0; j < kPairsAThread; ++j) {
            const uint32_t i = min(base + j * 256u + threadIdx.x, a.pairs - 1u);
            v[j] = a.indices[i];
            wv[j] = a.weights[i];
        }
#pragma unroll
        for (uint32_t j = 0; j < kPairsAThread; ++j) {
            const uint32_t i = base + j * 256u + threadIdx.x;
            if (i >= a.pairs) continue;
            if (v[j] < a.num_experts) atomicAdd(&s_hist[v[j]], 1u);
            if (in_lds) s_ids[i] = uint8_t(min(v[j], 255u));
            if (weights_in_lds) s_weights[i] = wv[j];
        }
    }
    __syncthreads();
    const uint32_t lane = threadIdx.x & 63u, e = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (e >= a.num_experts) return;
    // the keys and the residency word are fetched together, ahead of their use
    const uint64_t key = a.sort_keys ? a.sort_keys[e] : 0u;
    const uint64_t word = a.residency ? a.residency[e] : 0u;
    uint64_t other_key[SHRIKE_MAX_ROUTER_EXPERTS / 64u];
#pragma unroll
    for (uint32_t j = 0; j < SHRIKE_MAX_ROUTER_EXPERTS / 64u; ++j)
        other_key[j] = a.sort_keys ? a.sort_keys[min(lane + 64u * j, a.num_experts - 1u)] : 0u;
    uint32_t offset = 0, tiles_before = 0, tiles_total = 0;
#pragma unroll
    for (uint32_t j = 0; j < SHRIKE_MAX_ROUTER_EXPERTS / 64u; ++j) {
        const uint32_t other = lane + 64u * j;
        if (other >= a.num_experts) continue;
        const uint32_t c = s_hist[other];
        const uint64_t k2 = other_key[j];
        const bool before = k2 < key || (k2 == key && other < e);
        const uint32_t t = (c + kRowTile - 1u) / kRowTile;
        offset += before ? c : 0u;
        tiles_before += before ? t : 0u;
        tiles_total += t;
    }
    offset = wave_sum_u32(offset);
    tiles_before = wave_sum_u32(tiles_before);
    tiles_total = wave_sum_u32(tiles_total);
    const uint32_t count = s_hist[e];
    if (lane == 0) {
        a.counts[e] = count;
        a.offsets[e] = count ? offset : 0xffffffffu;
        if (e == 0) *a.tile_count = tiles_total;
    }
    uint32_t cell = e;
    if (a.residency)  // moe.metal:136-146
        cell = uint32_t(word >> 32) == SHRIKE_RESIDENCY_RESIDENT ? uint32_t(word) : kSentinel;
    const uint32_t my_tiles = (count + kRowTile - 1u) / kRowTile;
    for (uint32_t j = lane; j < my_tiles; j += 64u) {
        shrike_row_tile t;
        t.cell = cell;
        t.pair_start = offset + j * kRowTile;
        t.rows = min(kRowTile, count - j * kRowTile);
        t.expert = e;
        a.tiles[tiles_before + j] = t;
    }
    if (count == 0) return;
    // i / top_k == umulhi(i, magic) for i * top_k < 2^32; top_k == 1 would need magic 2^32, so it divides plainly below
    const uint32_t token_magic = 0xffffffffu / a.top_k + 1u;
    uint32_t running = 0;
    if (in_lds) {
        // 1,024 pairs a step: a lane takes 16 neighbouring ids with one LDS read, flags the bytes equal
        // to e, and a prefix sum over the lanes turns the per-lane counts into positions in index order
        const uint32_t pattern = e * 0x01010101u;
        for (uint32_t base = 0; base < a.pairs && running < count; base += 1024u) {
            const uint32_t i0 = base + lane * 16u;
            uint32_t match = 0;
            if (i0 < a.pairs) {
                const uint4 v = *reinterpret_cast<const uint4 *>(s_ids + i0);
                const uint32_t words[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const uint32_t x = words[w] ^ pattern;  // a zero byte where the id is e
                    const uint32_t t = ~(((x & 0x7f7f7f7fu) + 0x7f7f7f7fu) | x | 0x7f7f7f7fu);  // 0x80 in exactly those bytes
                    match |= ((((t >> 7) * 0x01020408u) >> 24) & 0xfu) << (4 * w);
                }
                const uint32_t valid = a.pairs - i0;  // ids past the last pair are whatever the LDS held
                if (valid < 16u) match &= (1u << valid) - 1u;
            }
            const uint32_t mine = __popc(match);
            const uint32_t upto = wave_inclusive_scan_u32(mine, lane);
            uint32_t at = offset + running + upto - mine;
            while (match) {
                const uint32_t i = i0 + uint32_t(__ffs(int(match)) - 1);
                match &= match - 1u;
                shrike_token_expert_pair p;
                p.token = a.top_k == 1u ? i : __umulhi(i, token_magic);
                p.expert = e;
                p.rank = i - p.token * a.top_k;
                p.weight_bits_and_reserved = weights_in_lds ? s_weights[i] : a.weights[i];
                if (at < offset + count) a.sorted[at] = p;  // ids the histogram did not count (out of range) never land
                ++at;
            }
            running += uint32_t(__builtin_amdgcn_readlane(int(upto), 63));
        }
        return;
    }
    const uint64_t below = (uint64_t(1) << lane) - 1u;
    for (uint32_t base = 0; base < a.pairs && running < count; base += 64u) {
        const uint32_t i = base + lane;
        const bool mine = i < a.pairs && a.indices[i] == e;
        const uint64_t mask = __ballot(mine);
        if (mine) {
            shrike_token_expert_pair p;
            p.token = a.top_k == 1u ? i : __umulhi(i, token_magic);
            p.expert = e;
            p.rank = i - p.token * a.top_k;
            p.weight_bits_and_reserved = a.weights[i];
            a.sorted[offset + running + __popcll(mask & below)] = p;
        }
        running += __popcll(mask);
    }
}

// ---- group sums -------------------------------------------------------------------------

// For every row of an fp16 matrix [rows, n] (row r at r * stride), the sum of each group of
// 64 elements, accumulated in fp32 in a fixed order and stored as two fp16 halves (hi, lo):
// the operand that turns the affine bias term sum_g bias[g] * (sum of x over g) into one
// more matrix product. Eight lanes share a group; a lane sums its eight elements in order,
// then the eight partials fold pairwise.
__global__ __launch_bounds__(256) void k_row_group_sums(const uint16_t *src, size_t stride, uint32_t rows, uint32_t n,
                                                        uint32_t *out, const uint32_t *row_limit_tiles) {
    const uint32_t groups = n / kGroup;
    const size_t slot = size_t(blockIdx.x) * 256u + threadIdx.x;  // (row, group, eighth)
    const size_t per_row = size_t(groups) * 8u;
    const uint32_t row = uint32_t(slot / per_row);
    uint32_t live_rows = rows;
    if (row_limit_tiles) live_rows = min(rows, *row_limit_tiles * kRowTile);
    const bool on = row < live_rows;
    const uint32_t rest = uint32_t(slot - size_t(row) * per_row);
    float s = 0.0f;
    if (on) {
        const uint4 v = *reinterpret_cast<const uint4 *>(src + size_t(row) * stride + size_t(rest) * 8u);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            s = __fadd_rn(s, f16_to_f32(uint16_t(w[t])));
            s = __fadd_rn(s, f16_to_f32(uint16_t(w[t] >> 16)));
        }
    }
    s = __fadd_rn(s, __shfl_xor(s, 1));
    s = __fadd_rn(s, __shfl_xor(s, 2));
    s = __fadd_rn(s, __shfl_xor(s, 4));
    if (on && (rest & 7u) == 0u) out[size_t(row) * groups + rest / 8u] = split_hi_lo(s);
}

// ---- reduce and residual ----------------------------------------------------------------

// prefill.metal:624-645: a thread owns eight neighbouring d of one token; fp32 fma in rank order
__global__ __launch_bounds__(256) void k_prefill_reduce(const uint16_t *partials, const uint16_t *weights, uint16_t *h2,
                                                        uint32_t query_count, uint32_t top_k, uint32_t d) {
    const uint32_t per_row = d / 8u;
    const size_t slot = size_t(blockIdx.x) * 256u + threadIdx.x;
    const uint32_t t = uint32_t(slot / per_row);
    if (t >= query_count) return;
    const uint32_t c = uint32_t(slot - size_t(t) * per_row);
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (uint32_t r = 0; r < top_k; ++r) {
        const float w = f16_to_f32(weights[size_t(t) * top_k + r]);
        const uint4 v = *reinterpret_cast<const uint4 *>(partials + (size_t(t) * top_k + r) * d + size_t(c) * 8u);
        const uint32_t p[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            acc[2 * j] = fmaf(w, f16_to_f32(uint16_t(p[j])), acc[2 * j]);
            acc[2 * j + 1] = fmaf(w, f16_to_f32(uint16_t(p[j] >> 16)), acc[2 * j + 1]);
        }
    }
    uint4 o;
    o.x = uint32_t(f32_to_f16(acc[0])) | uint32_t(f32_to_f16(acc[1])) << 16;
    o.y = uint32_t(f32_to_f16(acc[2])) | uint32_t(f32_to_f16(acc[3])) << 16;
    o.z = uint32_t(f32_to_f16(acc[4])) | uint32_t(f32_to_f16(acc[5])) << 16;
    o.w = uint32_t(f32_to_f16(acc[6])) | uint32_t(f32_to_f16(acc[7])) << 16;
    *reinterpret_cast<uint4 *>(h2 + size_t(t) * d + size_t(c) * 8u) = o;
}

__global__ __launch_bounds__(256) void k_residual_add(uint16_t *hidden, const uint16_t *delta, uint64_t count) {
    const uint64_t i = (uint64_t(blockIdx.x) * 256u + threadIdx.x) * 8u;
    if (i >= count) return;
    if (i + 8u <= count) {
        uint4 h = *reinterpret_cast<const uint4 *>(hidden + i);
        const uint4 dl = *reinterpret_cast<const uint4 *>(delta + i);
        uint32_t hw[4] = {h.x, h.y, h.z, h.w};
        const uint32_t dw[4] = {dl.x, dl.y, dl.z, dl.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint16_t lo = f32_to_f16(__fadd_rn(f16_to_f32(uint16_t(hw[j])), f16_to_f32(uint16_t(dw[j]))));
            const uint16_t hi = f32_to_f16(__fadd_rn(f16_to_f32(uint16_t(hw[j] >> 16)), f16_to_f32(uint16_t(dw[j] >> 16))));
            hw[j] = uint32_t(lo) | uint32_t(hi) << 16;
        }
        h.x = hw[0]; h.y = hw[1]; h.z = hw[2]; h.w = hw[3];
        *reinterpret_cast<uint4 *>(hidden + i) = h;
    } else {
        for (uint64_t j = i; j < count; ++j) hidden[j] = f32_to_f16(__fadd_rn(f16_to_f32(hidden[j]), f16_to_f32(delta[j])));
    }
}

// shared_scalar_gate_rows, moe.metal:1154-1193: one 8-bit group-affine weight row against a block of token rows,
// a workgroup a row. Eight partial sums as in the reference (its eight simdgroups of 32 lanes are the half-waves
// here): partial p takes the groups p, p + 8, ..., lane l of its 32 the elements 2l and 2l + 1 of a group; the 32
// lane sums fold by the butterfly 1, 2, 4, 8, 16 and the eight partials are added in index order.
__global__ __launch_bounds__(256) void k_scalar_gate_rows(const uint8_t *w, const uint16_t *scales, const uint16_t *biases,
                                                          uint32_t meta, const uint16_t *x, uint32_t x_stride, uint16_t *gate,
                                                          uint32_t d) {
    __shared__ float s_partial[8];
    const uint32_t p = threadIdx.x >> 5, l = threadIdx.x & 31u;
    const uint16_t *row = x + size_t(blockIdx.x) * x_stride;
    float acc = 0.0f;
    for (uint32_t g = p; g < d / kGroup; g += 8u) {
        const uint32_t i0 = g * kGroup + 2u * l;
        const uint32_t xw = *reinterpret_cast<const uint32_t *>(row + i0);
        const uint16_t qw = *reinterpret_cast<const uint16_t *>(w + i0);
        const float x0 = f16_to_f32(uint16_t(xw)), x1 = f16_to_f32(uint16_t(xw >> 16));
        const float dot = __fadd_rn(__fmul_rn(float(qw & 0xffu), x0), __fmul_rn(float(qw >> 8), x1));
        acc = fmaf(meta_f32(scales[g], meta), dot, acc);
        acc = fmaf(meta_f32(biases[g], meta), __fadd_rn(x0, x1), acc);
    }
#pragma unroll
    for (int o = 1; o <= 16; o <<= 1) acc = __fadd_rn(acc, __shfl_xor(acc, o));
    if (l == 0) s_partial[p] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        float total = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) total = __fadd_rn(total, s_partial[i]);
        gate[blockIdx.x] = f32_to_f16(total);
    }
}

// sigmoid_scalar_mul_rows_fp16, moe.metal:1195-1207: y[row, i] = half(y[row, i] / (1 + exp(-gate[row]))), eight
// elements a thread.
__global__ __launch_bounds__(256) void k_sigmoid_scalar_mul_rows(uint16_t *y, const uint16_t *gate, uint32_t d, uint32_t rows) {
    const uint32_t per_row = d / 8u;
    const uint64_t slot = uint64_t(blockIdx.x) * 256u + threadIdx.x;
    if (slot >= uint64_t(rows) * per_row) return;
    const uint32_t r = uint32_t(slot / per_row);
    const float div = 1.0f + expf(-f16_to_f32(gate[r]));
    uint4 v = *reinterpret_cast<const uint4 *>(y + slot * 8u);
    uint32_t vw[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint16_t lo = f32_to_f16(f16_to_f32(uint16_t(vw[j])) / div);
        const uint16_t hi = f32_to_f16(f16_to_f32(uint16_t(vw[j] >> 16)) / div);
        vw[j] = uint32_t(lo) | uint32_t(hi) << 16;
    }
    v.x = vw[0]; v.y = vw[1]; v.z = vw[2]; v.w = vw[3];
    *reinterpret_cast<uint4 *>(y + slot * 8u) = v;
}

int launch_row_group_sums(const uint16_t *src, size_t stride, uint32_t rows, uint32_t n, uint32_t *out,
                          const uint32_t *row_limit_tiles, hipStream_t s) {
    const size_t slots = size_t(rows) * (n / kGroup) * 8u;
    if (slots == 0) return 0;
    hipLaunchKernelGGL(k_row_group_sums, dim3(uint32_t((slots + 255u) / 256u)), dim3(256), 0, s, src, stride, rows, n, out,
                       row_limit_tiles);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

}  // namespace shrike

using namespace shrike;

// d_group_sums (may be null): where the group sums of hidden's rows go as well, for the grouped FFN's bias term
static int prefill_router(shrike_hip_moe *moe, void *stream, const void *d_weights, const void *d_scales, const void *d_biases,
                          const void *d_hidden, const void *d_effective_scale, const void *d_per_expert_scale,
                          const void *d_logit_bias, uint32_t *d_out_indices, void *d_out_weights, float *d_logits_workspace,
                          uint32_t query_count, uint32_t num_experts, uint32_t d, uint32_t top_k, uint32_t hidden_stride_elements,
                          uint32_t *d_group_sums) {
    SHRIKE_REQUIRE(moe != nullptr, "moe handle is NULL");
    SHRIKE_REQUIRE(query_count > 0, "queryCount must be positive");  // PrefillRouter.swift:99
    if (int rc = check_router(moe, num_experts, d, top_k)) return rc;
    SHRIKE_REQUIRE(hidden_stride_elements >= d, "hidden stride is too small");  // PrefillRouter.swift:104
    SHRIKE_REQUIRE(hidden_stride_elements % 8u == 0, "hidden stride must keep rows 16-byte aligned");
    SHRIKE_REQUIRE(d_weights && d_hidden && d_effective_scale && d_per_expert_scale && d_logit_bias,
                   "prefill router: weights, hidden, effectiveScale, perExpertScale and logitBias must all be bound");
    SHRIKE_REQUIRE(moe->desc.router_weight_bits == 0 || (d_scales && d_biases), "prefill router: affine router needs scales and biases");
    SHRIKE_REQUIRE(d_out_indices && d_out_weights && d_logits_workspace, "prefill router: outputs and the workspace must be bound");
    SHRIKE_REQUIRE(reinterpret_cast<uintptr_t>(d_logits_workspace) % 16u == 0, "prefill router: workspace must be 16-byte aligned");
    RouterArgs a = {};
    a.weights = d_weights;
    a.scales = static_cast<const uint16_t *>(d_scales);
    a.biases = static_cast<const uint16_t *>(d_biases);
    a.hidden = static_cast<const uint16_t *>(d_hidden);
    a.effective_scale = static_cast<const uint16_t *>(d_effective_scale);
    a.d = d;
    a.meta = moe->desc.meta_dtype;
    a.sel.per_expert_scale = static_cast<const uint16_t *>(d_per_expert_scale);
    a.sel.logit_bias = static_cast<const uint16_t *>(d_logit_bias);
    a.sel.num_experts = num_experts;
    a.sel.top_k = top_k;
    a.sel.sigmoid = moe->desc.sigmoid_router_scores;
    a.sel.scaling = moe->desc.routed_scaling_factor;
    hipStream_t s = as_stream(stream);
    if (query_count <= kRouterLaunchTokens) {
        // a handful of tokens (decode for several sequences): the decode router's kernel with the tokens
        // on the grid, one launch for logits and selection instead of three
        a.logits_out = d_logits_workspace;
        a.sel.logits = d_logits_workspace;
        a.lists.out_indices = d_out_indices;
        a.lists.out_weights = static_cast<uint16_t *>(d_out_weights);
        a.counter = moe->d_counter + kRouterTokenCounters;
        a.token_stride = hidden_stride_elements;
        if (int rc = launch_router_tokens(a, moe->desc.router_weight_bits, query_count, s)) return rc;
        return d_group_sums ? launch_row_group_sums(a.hidden, hidden_stride_elements, query_count, d, d_group_sums, nullptr, s) : 0;
    }
    const dim3 grid((num_experts + 3u) / 4u, (query_count + kRouterTokenBlock - 1u) / kRouterTokenBlock);
    switch (moe->desc.router_weight_bits) {
        case 0: {
            // four packed rows a wave where a row is four chunks a lane, two where it is up to eight
            const uint16_t *w16 = static_cast<const uint16_t *>(d_weights);
            if (d <= 2048u)
                launch_prefill_logits_f16<4, 4>(w16, a.hidden, hidden_stride_elements, a.effective_scale, d_logits_workspace, query_count,
                                                num_experts, d, s);
            else
                launch_prefill_logits_f16<8, 2>(w16, a.hidden, hidden_stride_elements, a.effective_scale, d_logits_workspace, query_count,
                                                num_experts, d, s);
            break;
        }
        case 8: hipLaunchKernelGGL(k_prefill_logits<8>, grid, dim3(256), 0, s, a, query_count, hidden_stride_elements, d_logits_workspace); break;
        default: hipLaunchKernelGGL(k_prefill_logits<4>, grid, dim3(256), 0, s, a, query_count, hidden_stride_elements, d_logits_workspace); break;
    }
    SHRIKE_HIP(hipGetLastError());
    if (d_group_sums)  // the selection's waves form them on the side
        hipLaunchKernelGGL(k_prefill_select<true>, dim3((query_count + 3u) / 4u), dim3(256), 0, s, a.sel, d_logits_workspace,
                           d_out_indices, static_cast<uint16_t *>(d_out_weights), query_count, a.hidden, hidden_stride_elements, d,
                           d_group_sums);
    else
        hipLaunchKernelGGL(k_prefill_select<false>, dim3((query_count + 3u) / 4u), dim3(256), 0, s, a.sel, d_logits_workspace,
                           d_out_indices, static_cast<uint16_t *>(d_out_weights), query_count, a.hidden, hidden_stride_elements, d,
                           nullptr);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

extern "C" {

int shrike_hip_prefill_router(shrike_hip_moe *moe, void *stream, const void *d_weights, const void *d_scales,
                              const void *d_biases, const void *d_hidden, const void *d_effective_scale,
                              const void *d_per_expert_scale, const void *d_logit_bias, uint32_t *d_out_indices,
                              void *d_out_weights, float *d_logits_workspace, uint32_t query_count, uint32_t num_experts,
                              uint32_t d, uint32_t top_k, uint32_t hidden_stride_elements) {
    return prefill_router(moe, stream, d_weights, d_scales, d_biases, d_hidden, d_effective_scale, d_per_expert_scale, d_logit_bias,
                          d_out_indices, d_out_weights, d_logits_workspace, query_count, num_experts, d, top_k,
                          hidden_stride_elements, nullptr);
}

int shrike_hip_prefill_router_with_group_sums(shrike_hip_moe *moe, void *stream, const void *d_weights, const void *d_scales,
                                              const void *d_biases, const void *d_hidden, const void *d_effective_scale,
                                              const void *d_per_expert_scale, const void *d_logit_bias,
                                              uint32_t *d_out_indices, void *d_out_weights, float *d_logits_workspace,
                                              uint32_t query_count, uint32_t num_experts, uint32_t d, uint32_t top_k,
                                              uint32_t hidden_stride_elements, void *d_ffn_workspace) {
    SHRIKE_REQUIRE(d_ffn_workspace != nullptr, "prefill router: the FFN workspace that takes the group sums is NULL");
    SHRIKE_REQUIRE(reinterpret_cast<uintptr_t>(d_ffn_workspace) % 256u == 0, "prefill router: the FFN workspace must be 256-byte aligned");
    SHRIKE_REQUIRE(d % kGroup == 0, "prefill router: group sums need d to be a multiple of 64, got %u", d);
    return prefill_router(moe, stream, d_weights, d_scales, d_biases, d_hidden, d_effective_scale, d_per_expert_scale, d_logit_bias,
                          d_out_indices, d_out_weights, d_logits_workspace, query_count, num_experts, d, top_k,
                          hidden_stride_elements, static_cast<uint32_t *>(d_ffn_workspace));
}

size_t shrike_hip_prefill_router_workspace_bytes(uint32_t query_count, uint32_t num_experts, uint32_t d) {
    (void)d;  // the fp32 logits alone: x times the effective scale is formed inside the logits kernel
    return ((size_t(query_count) * num_experts + 3u) & ~size_t(3)) * sizeof(float);
}

uint32_t shrike_hip_group_max_row_tiles(uint64_t pair_count, uint32_t num_experts) {
    return max_row_tiles(pair_count, num_experts);
}

int shrike_hip_group_pairs(void *stream, const uint32_t *d_indices, const void *d_weights, uint32_t query_count,
                           uint32_t top_k, uint32_t num_experts, const uint64_t *d_expert_sort_keys,
                           const uint64_t *d_residency, const shrike_hip_grouped_routes *out) {
    SHRIKE_REQUIRE(top_k > 0, "topK must be positive, got %u", top_k);                    // PrefillMoEGrouping.swift:280
    SHRIKE_REQUIRE(num_experts > 0, "numExperts must be positive, got %u", num_experts);  // :283
    SHRIKE_REQUIRE(num_experts <= SHRIKE_MAX_ROUTER_EXPERTS, "numExperts > 256 is not supported");
    SHRIKE_REQUIRE(uint64_t(query_count) * top_k <= 0x7fffffffull, "too many route pairs");
    SHRIKE_REQUIRE(out && out->sorted_pairs && out->per_expert_offsets && out->per_expert_counts && out->row_tiles && out->row_tile_count,
                   "group pairs: an output is NULL");
    SHRIKE_REQUIRE(query_count == 0 || (d_indices && d_weights), "group pairs: indices and weights must be bound");
    GroupArgs a = {};
    a.indices = d_indices;
    a.weights = static_cast<const uint16_t *>(d_weights);
    a.pairs = query_count * top_k;
    a.top_k = top_k;
    a.num_experts = num_experts;
    a.sort_keys = d_expert_sort_keys;
    a.residency = d_residency;
    a.sorted = static_cast<shrike_token_expert_pair *>(out->sorted_pairs);
    a.offsets = out->per_expert_offsets;
    a.counts = out->per_expert_counts;
    a.tiles = out->row_tiles;
    a.tile_count = out->row_tile_count;
    hipStream_t s = as_stream(stream);
    const dim3 grid((num_experts + 3u) / 4u);
    hipLaunchKernelGGL(k_group, grid, dim3(256), 0, s, a);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

int shrike_hip_shared_scalar_gate_rows(void *stream, const shrike_projection *gate_row, uint32_t meta_dtype, const void *d_x,
                                       uint32_t x_stride_elements, void *d_gate, uint32_t rows, uint32_t d) {
    SHRIKE_REQUIRE(gate_row && gate_row->weights && gate_row->scales && gate_row->biases, "scalar gate rows: the gate row must be bound");
    SHRIKE_REQUIRE(d_x && d_gate, "scalar gate rows: NULL buffer");
    // Elementwise.swift:148
    SHRIKE_REQUIRE(d > 0 && d % SHRIKE_GROUP_SIZE == 0, "shared_scalar_gate_rows drops the tail unless d is a multiple of 64");
    SHRIKE_REQUIRE(x_stride_elements >= d && x_stride_elements % 2u == 0, "scalar gate rows: x stride is too small or odd");
    SHRIKE_REQUIRE(meta_dtype <= SHRIKE_META_F16, "scalar gate rows: metaDtype=%u is not a known value", meta_dtype);
    if (rows == 0) return 0;
    hipLaunchKernelGGL(k_scalar_gate_rows, dim3(rows), dim3(256), 0, as_stream(stream), static_cast<const uint8_t *>(gate_row->weights),
                       static_cast<const uint16_t *>(gate_row->scales), static_cast<const uint16_t *>(gate_row->biases), meta_dtype,
                       static_cast<const uint16_t *>(d_x), x_stride_elements, static_cast<uint16_t *>(d_gate), d);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

int shrike_hip_sigmoid_scalar_mul_rows(void *stream, void *d_y, const void *d_gate, uint32_t d, uint32_t rows) {
    SHRIKE_REQUIRE(d_y && d_gate, "sigmoid scalar mul rows: NULL buffer");
    SHRIKE_REQUIRE(d % 8u == 0 && reinterpret_cast<uintptr_t>(d_y) % 16u == 0, "sigmoid scalar mul rows: d must be a multiple of 8 and y 16-byte aligned");
    const uint64_t slots = uint64_t(rows) * (d / 8u);
    if (slots == 0) return 0;
    hipLaunchKernelGGL(k_sigmoid_scalar_mul_rows, dim3(uint32_t((slots + 255u) / 256u)), dim3(256), 0, as_stream(stream),
                       static_cast<uint16_t *>(d_y), static_cast<const uint16_t *>(d_gate), d, rows);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

int shrike_hip_prefill_reduce(void *stream, const void *d_route_partials, const void *d_route_weights, void *d_h2,
                              uint32_t query_count, uint32_t top_k, uint32_t d) {
    SHRIKE_REQUIRE(d_route_partials && d_route_weights && d_h2, "prefill reduce: NULL buffer");
    SHRIKE_REQUIRE(d % 8u == 0 && top_k > 0, "prefill reduce: D must be a multiple of 8 and topK positive");
    const size_t slots = size_t(query_count) * (d / 8u);
    if (slots == 0) return 0;
    hipLaunchKernelGGL(k_prefill_reduce, dim3(uint32_t((slots + 255u) / 256u)), dim3(256), 0, as_stream(stream),
                       static_cast<const uint16_t *>(d_route_partials), static_cast<const uint16_t *>(d_route_weights),
                       static_cast<uint16_t *>(d_h2), query_count, top_k, d);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

int shrike_hip_residual_add_f16(void *stream, void *d_hidden, const void *d_delta, uint64_t count) {
    SHRIKE_REQUIRE(d_hidden && d_delta, "residual add: NULL buffer");
    SHRIKE_REQUIRE((reinterpret_cast<uintptr_t>(d_hidden) | reinterpret_cast<uintptr_t>(d_delta)) % 16u == 0,
                   "residual add: buffers must be 16-byte aligned");
    if (count == 0) return 0;
    const uint64_t threads = (count + 7u) / 8u;
    hipLaunchKernelGGL(k_residual_add, dim3(uint32_t((threads + 255u) / 256u)), dim3(256), 0, as_stream(stream),
                       static_cast<uint16_t *>(d_hidden), static_cast<const uint16_t *>(d_delta), count);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

}  // extern "C"
