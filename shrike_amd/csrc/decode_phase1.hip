// Phase 1 of the routed decode layer for gfx950: gate and up matvecs of the selected
// experts against one activation vector, GLU, fp16 activations out
// (moe.metal:950-999 for 4-bit codes, the :650-672 body for 8-bit, pool addressing
// :297-305). In the fused layer the same launch routes (select + classify in the prologue
// of every workgroup, from the logits of the previous launch) and carries the shared
// expert's down projection in extra workgroups.
#include "decode_launch.h"

namespace shrike {

constexpr int kPhase1RowPairs = 4;  // (gate, up) row pairs per wave
// ... and in a launch that does not route, for one token or for rows of three or more 16-byte chunks a lane: twice the
// waves with half the rows in flight each measured faster there (one token 5.06 -> 4.68 us at hidden 2048, a batch of
// four tokens at hidden 2880 with 8-bit codes 84 -> 79 us a layer; the same batch with 4-bit codes is slower with them)
constexpr int kPhase1RowPairsNarrow = 2;

// A wave owns RP consecutive f of one routed position: RP gate rows and RP up rows, each a
// run of 16-byte chunks across the lanes. The lane's slice of x comes straight from global
// memory (L2-resident) ahead of the row loads, so in-order load return never holds it back.
// STREAM: one token, so every routed row is read exactly once: the row loads are non-temporal (a batch of tokens
// reads an expert's rows once per token routed to it, and there the caches are what makes the second read cheap).
// TAIL: the rows end in a step of half chunks (load_slice_regs); NCH then counts the whole steps ahead of it.
// META: the type of the routed experts' scales and biases (SHRIKE_META_*), known to the instance so that a row converts them one way.
template <int BITS, int NCH, int RP, bool ROUTE, int SBITS, bool STREAM, bool TAIL, int META>
__global__ __launch_bounds__(256) void k_phase1(Phase1Args a) {
    warm_kernel_arguments(a);
    typedef Chunk<BITS> C;
    if (ROUTE && blockIdx.x == a.lists_block) {
        // the workgroup behind all others: one wave selects once more and writes what the host and phase 2 read
        // (indices, weights, hit and miss lists, resolved cells); nobody in this launch waits for it. With a batch of
        // tokens (grid.y) each token has one, writing its own top_k indices, weights and cells.
        if (threadIdx.x < 64u) {
            const size_t t_ = blockIdx.y;
            const TableSelect t = select_from_table(a.route_table + t_ * SHRIKE_MAX_ROUTER_EXPERTS, a.sel.num_experts, a.sel.top_k,
                                                    threadIdx.x, a.sel.top_k);
            RouteLists lists = a.lists;
            lists.out_indices = a.lists.out_indices + t_ * a.top_k;
            lists.out_weights = a.lists.out_weights + t_ * a.top_k;
            lists.resolved_slots = a.lists.resolved_slots + t_ * a.top_k;
            uint32_t my_cell;
            finish_routes(a.sel, lists, threadIdx.x, true, t.mine, t.my_key, t.my_raw, bf16_to_f32(uint16_t(t.my_gain)),
                          t.my_cell, my_cell);
        }
        return;
    }
    if (SBITS != 0 && blockIdx.x >= a.routed_blocks) {
        gemv_job<SBITS == 0 ? 4 : SBITS, 1>(a.shared_down, blockIdx.x - a.routed_blocks);
        return;
    }
    if (a.indirect && a.indirect[0] == 0u) return;
    if (!io_ready(a.io_status)) return;
    // a batch of tokens: grid.y is this workgroup's token (the argument block itself stays untouched:
    // writing to it would move it to private memory)
    const size_t tok = blockIdx.y;
    const uint16_t *x_tok = a.x + tok * a.x_stride;
    const uint32_t *resolved_tok = a.resolved + tok * a.top_k;
    uint16_t *acts_tok = a.acts + tok * a.top_k * a.f;
    const uint32_t lane = threadIdx.x & 63u, wave = wave_index();
    const uint32_t cpr = a.d * BITS / 128u, groups = a.d / kGroup, row_bytes = cpr * 16u;
    const uint32_t pair0 = (blockIdx.x * 4u + wave) * RP;
    bool in_range = pair0 < (a.active ? a.active_count : a.top_k) * a.f;
    uint32_t k = in_range ? pair0 / a.f : 0u;
    const uint32_t f0 = pair0 - k * a.f;
    if (!ROUTE && a.active) {  // moe.metal:873-876: the wave's position comes from the list; one past top_k is skipped
        k = in_range ? a.active[k] : 0u;
        in_range = in_range && k < a.top_k;
        k = in_range ? k : 0u;
    }

    uint32_t cell = kSentinel;
    SliceRegs<BITS, NCH, TAIL> xr;
    if (ROUTE) {
        // every wave selects for itself, in registers, from the table the previous launch left: no barrier, and the
        // table's loads go out ahead of the activation slice's (loads return in order)
        // (a wave stops at the round that names its own position's expert)
        const TableSelect t = select_from_table(a.route_table + tok * SHRIKE_MAX_ROUTER_EXPERTS, a.sel.num_experts, a.sel.top_k, lane, k);
        load_slice_regs<BITS, NCH, TAIL>(xr, reinterpret_cast<const uint4 *>(x_tok), cpr, lane, true);
        if (in_range) cell = uint32_t(__builtin_amdgcn_readlane(int(t.my_cell), int(k)));
    } else {
        load_slice_regs<BITS, NCH, TAIL>(xr, reinterpret_cast<const uint4 *>(x_tok), cpr, lane, true);
        if (in_range && !a.blobs) cell = resolved_tok[k];
    }
    const uint8_t *base;
    if (!ROUTE && a.blobs) {  // moe.metal:821: the blob the argument buffer names for this position
        base = in_range ? a.blobs[k] : nullptr;
        if (base == nullptr) return;
    } else {
        if (cell == kSentinel) return;  // moe.metal:986, and waves past the last row
        base = cell_base_uniform(a.pool, cell, a.stride);
    }

    RowRegs<BITS, NCH, TAIL> rows[2 * RP];
#pragma unroll
    for (int r = 0; r < 2 * RP; ++r) {
        const bool up = r >= RP;
        const uint32_t f = f0 + uint32_t(r % RP);
        const uint8_t *w = base + (up ? a.off.up_w_off : a.off.gate_w_off) + size_t(f) * row_bytes;
        const uint16_t *s = reinterpret_cast<const uint16_t *>(base + (up ? a.off.up_s_off : a.off.gate_s_off)) + size_t(f) * groups;
        const uint16_t *b = reinterpret_cast<const uint16_t *>(base + (up ? a.off.up_b_off : a.off.gate_b_off)) + size_t(f) * groups;
        load_row<BITS, NCH, STREAM, TAIL>(rows[r], w, s, b, cpr, lane, true);
    }
    float gab = 0.0f, uab = 0.0f;
    if (a.ebias && lane < uint32_t(RP)) {  // moe.metal:261-269
        gab = bf16_to_f32(reinterpret_cast<const uint16_t *>(base + a.off.gate_ab_off)[f0 + lane]);
        uab = bf16_to_f32(reinterpret_cast<const uint16_t *>(base + a.off.up_ab_off)[f0 + lane]);
    }

    typename C::X x[NCH];
    float xs[NCH];
    TailX xt;
    unpack_slices<BITS, NCH, TAIL>(xr, x, xs, xt);
    float res[2 * RP];
#pragma unroll
    for (int r = 0; r < 2 * RP; ++r) res[r] = wave_sum(row_partial<BITS, NCH, TAIL>(rows[r], x, xs, xt, uint32_t(META)));
    // lane p < RP finishes row pair p
    float g = res[0], u = res[RP];
#pragma unroll
    for (int p = 1; p < RP; ++p) {
        g = lane == uint32_t(p) ? res[p] : g;
        u = lane == uint32_t(p) ? res[RP + p] : u;
    }
    const uint16_t act = f32_to_f16(glu_rt(g + gab, u + uab, a.act));
    if (lane < uint32_t(RP)) acts_tok[size_t(k) * a.f + f0 + lane] = act;
}

// positions: top_k, or the length of the active list
static uint32_t phase1_blocks_of(uint32_t positions, uint32_t f, uint32_t row_pairs) {
    const uint32_t waves = (positions * f + row_pairs - 1) / row_pairs;
    return (waves + 3) / 4;
}
uint32_t phase1_blocks(uint32_t top_k, uint32_t f) { return phase1_blocks_of(top_k, f, kPhase1RowPairs); }

// (a row that ends in half chunks counts the steps it would take without them: the choice stays what it was measured as)
static bool phase1_narrow(bool routing, bool one_token, uint32_t d, uint32_t bits) {
    return one_token ? !routing : nch_for(d, bits) >= 3;
}

template <int BITS, bool ROUTE, int SBITS, bool STREAM, int META>
static void launch_phase1_meta(const Phase1Args &a, dim3 grid, hipStream_t s) {
    // (the one-token routing launch keeps four pairs; a batch takes the narrow form for long rows whether it routes or not)
    constexpr int RP = kPhase1RowPairs, RN = (ROUTE && STREAM) ? kPhase1RowPairs : kPhase1RowPairsNarrow;
    const dim3 block(256);
    if (BITS == 4 && half_chunk_tail(a.d * BITS / 128u, BITS)) {
        // d <= SHRIKE_MAX_HIDDEN: one whole step and the half chunks (65...96 chunks a row)
        hipLaunchKernelGGL((k_phase1<BITS, 1, STREAM ? RN : RP, ROUTE, SBITS, STREAM, BITS == 4, META>), grid, block, 0, s, a);
        return;
    }
    switch (nch_for(a.d, BITS)) {
        case 1: hipLaunchKernelGGL((k_phase1<BITS, 1, STREAM ? RN : RP, ROUTE, SBITS, STREAM, false, META>), grid, block, 0, s, a); break;
        case 2: hipLaunchKernelGGL((k_phase1<BITS, 2, STREAM ? RN : RP, ROUTE, SBITS, STREAM, false, META>), grid, block, 0, s, a); break;
        case 3: hipLaunchKernelGGL((k_phase1<BITS, 3, RN, ROUTE, SBITS, STREAM, false, META>), grid, block, 0, s, a); break;
        default: hipLaunchKernelGGL((k_phase1<BITS, 4, RN, ROUTE, SBITS, STREAM, false, META>), grid, block, 0, s, a); break;
    }
}

template <int BITS, bool ROUTE, int SBITS, bool STREAM>
static void launch_phase1_nch(const Phase1Args &a, dim3 grid, hipStream_t s) {
    if (a.meta == SHRIKE_META_F16) launch_phase1_meta<BITS, ROUTE, SBITS, STREAM, SHRIKE_META_F16>(a, grid, s);
    else launch_phase1_meta<BITS, ROUTE, SBITS, STREAM, SHRIKE_META_BF16>(a, grid, s);
}

int launch_phase1(const Phase1Args &a, uint32_t bits, bool routing, uint32_t shared_down_bits, hipStream_t s) {
    SHRIKE_REQUIRE(a.f % kPhase1RowPairs == 0, "phase1: f=%u must be a multiple of %d", a.f, kPhase1RowPairs);
    uint32_t extra = 0;
    SHRIKE_REQUIRE(a.tokens <= 1u || shared_down_bits == 0, "phase1: the shared down rows ride along with one token only");
    if (shared_down_bits) {
        SHRIKE_REQUIRE(routing && nch_for(a.shared_down.n, shared_down_bits) == 1,
                       "phase1: the shared down rows ride along only in the routed launch and with one chunk column per lane");
        extra = gemv_blocks(a.shared_down.rows, a.shared_down.n, shared_down_bits);
    }
    Phase1Args b = a;
    const bool one_token = a.tokens <= 1u;
    if (phase1_narrow(routing, one_token, a.d, bits))
        b.routed_blocks = phase1_blocks_of(a.active ? a.active_count : a.top_k, a.f, kPhase1RowPairsNarrow);
    b.lists_block = routing ? b.routed_blocks + extra : 0xffffffffu;
    const dim3 grid(b.routed_blocks + extra + (routing ? 1u : 0u), a.tokens ? a.tokens : 1u);
    if (bits == 4) {
        if (!routing) { if (one_token) launch_phase1_nch<4, false, 0, true>(b, grid, s); else launch_phase1_nch<4, false, 0, false>(b, grid, s); }
        else if (shared_down_bits == 0) { if (one_token) launch_phase1_nch<4, true, 0, true>(b, grid, s); else launch_phase1_nch<4, true, 0, false>(b, grid, s); }
        else if (shared_down_bits == 4) launch_phase1_nch<4, true, 4, true>(b, grid, s);
        else launch_phase1_nch<4, true, 8, true>(b, grid, s);
    } else {
        if (!routing) { if (one_token) launch_phase1_nch<8, false, 0, true>(b, grid, s); else launch_phase1_nch<8, false, 0, false>(b, grid, s); }
        else if (shared_down_bits == 0) { if (one_token) launch_phase1_nch<8, true, 0, true>(b, grid, s); else launch_phase1_nch<8, true, 0, false>(b, grid, s); }
        else if (shared_down_bits == 4) launch_phase1_nch<8, true, 4, true>(b, grid, s);
        else launch_phase1_nch<8, true, 8, true>(b, grid, s);
    }
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

int check_offsets(const shrike_expert_offsets *o, uint32_t d, uint32_t f, uint32_t bits) {
    SHRIKE_REQUIRE(o != nullptr, "offsets is NULL");
    SHRIKE_REQUIRE(d % SHRIKE_GROUP_SIZE == 0 && f % SHRIKE_GROUP_SIZE == 0,
                   "d=%u and f=%u must be multiples of %u", d, f, SHRIKE_GROUP_SIZE);
    SHRIKE_REQUIRE(d <= SHRIKE_MAX_HIDDEN, "d=%u exceeds the activation ceiling %u", d, SHRIKE_MAX_HIDDEN);
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

}  // namespace shrike

using namespace shrike;

extern "C" {

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
    return launch_phase1(a, bits, false, 0, as_stream(stream));
}

int shrike_hip_moe_phase1_blobs(shrike_hip_moe *moe, void *stream, const void *const *d_routed_blobs,
                                const shrike_expert_offsets *offsets, const void *d_x, void *d_acts, uint32_t d, uint32_t f,
                                uint32_t top_k, const uint32_t *d_active_slots, uint32_t active_count,
                                const uint32_t *d_io_status) {
    SHRIKE_REQUIRE(moe != nullptr, "moe handle is NULL");
    SHRIKE_REQUIRE(top_k >= 1 && top_k <= SHRIKE_MAX_TOP_K, "phase1: topK=%u not in 1...8", top_k);  // MoE.validate(routedBlobs:topK:)
    const uint32_t bits = moe->desc.routed_weight_bits;
    if (int rc = check_offsets(offsets, d, f, bits)) return rc;
    SHRIKE_REQUIRE(d_routed_blobs && d_x && d_acts, "phase1: the argument buffer, x and acts must be bound");
    if (d_active_slots != nullptr && active_count == 0) return 0;  // MoE.swift:710: nothing to do is not an error
    SHRIKE_REQUIRE(d_active_slots != nullptr || active_count == 0, "phase1: activeCount=%u without an active list", active_count);
    SHRIKE_REQUIRE(active_count <= SHRIKE_MAX_TOP_K, "phase1: activeCount=%u exceeds %u", active_count, SHRIKE_MAX_TOP_K);
    Phase1Args a = {};
    a.blobs = reinterpret_cast<const uint8_t *const *>(d_routed_blobs);
    a.active = d_active_slots; a.active_count = active_count;
    a.off = *offsets;
    a.x = static_cast<const uint16_t *>(d_x); a.acts = static_cast<uint16_t *>(d_acts);
    a.d = d; a.f = f; a.top_k = top_k; a.meta = moe->desc.meta_dtype; a.act = moe->desc.activation;
    a.ebias = moe->desc.expert_additive_biases;
    a.io_status = moe->desc.event_gated_io ? d_io_status : nullptr;
    a.resolved = nullptr;
    a.routed_blocks = phase1_blocks(d_active_slots ? active_count : top_k, f);
    return launch_phase1(a, bits, false, 0, as_stream(stream));
}

int shrike_hip_moe_phase1_batch(shrike_hip_moe *moe, void *stream, const shrike_pool_bases *pool,
                                uint64_t pool_slot_stride, const uint32_t *d_resolved_slots,
                                const shrike_expert_offsets *offsets, const void *d_x, uint32_t x_stride_elements,
                                void *d_acts, uint32_t d, uint32_t f, uint32_t top_k, uint32_t tokens) {
    SHRIKE_REQUIRE(moe != nullptr && pool != nullptr, "moe handle or pool is NULL");
    SHRIKE_REQUIRE(top_k >= 1 && top_k <= SHRIKE_MAX_TOP_K, "phase1: topK=%u not in 1...8", top_k);
    SHRIKE_REQUIRE(tokens >= 1 && tokens <= 65535u, "phase1: %u tokens not in 1...65535", tokens);
    SHRIKE_REQUIRE(x_stride_elements >= d && x_stride_elements % 8u == 0, "phase1: x stride is too small or leaves rows unaligned");
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
    a.tokens = tokens; a.x_stride = x_stride_elements;
    a.routed_blocks = phase1_blocks(top_k, f);
    return launch_phase1(a, bits, false, 0, as_stream(stream));
}

}  // extern "C"
