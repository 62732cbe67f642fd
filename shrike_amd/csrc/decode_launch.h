// Argument blocks and launchers of the decode kernels, shared by the translation units
// that define them and by the fused-layer entry point.
#pragma once

#include "gemv_common.h"

namespace shrike {

struct RouterArgs {
    const void *weights;
    const uint16_t *scales, *biases;
    const uint16_t *hidden, *effective_scale;
    uint32_t d, meta;
    uint32_t *counter;
    float *logits_out;
    SelectArgs sel;
    RouteLists lists;  // out_indices == nullptr: logits only
    RouteEntry *route_table;  // head launch of the fused layer: one entry per expert beside the logit (lists.residency read)
    // several tokens in one launch (grid.y): token t reads hidden + t * token_stride, writes logits_out + t *
    // num_experts and out_indices / out_weights + t * top_k, and counts arrivals in counter[t]; select only
    uint32_t token_stride;
};

struct Phase1Args {
    PoolArg pool;
    uint64_t stride;
    const uint32_t *resolved;
    shrike_expert_offsets off;
    const uint16_t *x;
    uint16_t *acts;
    uint32_t d, f, top_k, meta, act, ebias;
    const uint32_t *indirect, *io_status;
    uint32_t tokens, x_stride;  // tokens > 1: grid.y walks tokens; x rows x_stride elements apart
    // argument-buffer addressing (moe.metal:779-884): position k's blob is blobs[k] in place of a pool cell; with
    // `active` bound only the positions active[0 .. active_count) are computed, the grid covering active_count * f rows
    const uint8_t *const *blobs;
    const uint32_t *active;
    uint32_t active_count;
    // fused layer only: every wave selects from the route table the previous launch left, the shared expert's down
    // projection runs in workgroups past `routed_blocks`, and one more workgroup behind those writes the route lists
    SelectArgs sel;
    RouteLists lists;
    const RouteEntry *route_table;
    uint32_t lists_block;  // set by launch_phase1: the workgroup that writes the route lists
    uint32_t routed_blocks;
    GemvArgs shared_down;
};

struct Phase2Args {
    PoolArg pool;
    uint64_t stride;
    const uint32_t *resolved, *fallback;
    shrike_expert_offsets off;
    const uint16_t *acts, *routing_w, *residual;
    uint16_t *y, *hidden;
    uint32_t d, f, top_k, meta, ebias;
    const uint32_t *indirect, *io_status;
    uint32_t tokens;  // tokens > 1: grid.y walks tokens; residual, y and hidden rows are d apart
    const uint8_t *const *blobs;  // argument-buffer addressing (moe.metal:897-941): position k's blob, in place of a pool cell
    const uint16_t *delta;  // fp16[d] or null: hidden = half(half(hidden + delta) + y), the residual add of a norm fused ahead
};

// The residual add + RMS norm ahead of the layer, done by every workgroup of the head launch for itself:
// x = norm(hidden + delta) * weight. hidden is read only (phase 2 applies the add); the first workgroup
// stores x to x_out for the launches that follow.
struct NormArgs {
    const uint16_t *hidden, *delta, *weight;
    uint16_t *x_out;
    float eps;
};

int launch_router(const RouterArgs &a, uint32_t router_bits, hipStream_t s);
// the same for `tokens` tokens in one launch; a.counter must have a zeroed word for each
constexpr uint32_t kRouterLaunchTokens = 16;  // up to here the one-launch router beats the three-launch prefill router
int launch_router_tokens(const RouterArgs &a, uint32_t router_bits, uint32_t tokens, hipStream_t s);
// router logit rows + the shared expert's gate/up rows in one grid
// norm: null, or the norm to run in every workgroup's prologue (r.hidden and g.x are then not read)
// tokens > 1 (router rows only): grid.y walks tokens, token t reading r.hidden + t * r.token_stride and writing the t-th
// logit row and route table (SHRIKE_MAX_ROUTER_EXPERTS entries apart)
int launch_head(const RouterArgs &r, uint32_t router_bits, const GemvArgs &g, uint32_t shared_bits, const NormArgs *norm, hipStream_t s,
                uint32_t tokens = 1);
uint32_t phase1_blocks(uint32_t top_k, uint32_t f);
// shared_down_bits: 0 = none, else the shared down rows ride in the same grid (one chunk
// column per lane only: nch_for(shared_f, bits) == 1)
int launch_phase1(const Phase1Args &a, uint32_t bits, bool routing, uint32_t shared_down_bits, hipStream_t s);
int launch_phase2(const Phase2Args &a, uint32_t bits, hipStream_t s);
int launch_gemv(const GemvArgs &a, uint32_t bits, hipStream_t s);

int check_offsets(const shrike_expert_offsets *o, uint32_t d, uint32_t f, uint32_t bits);
int check_router(const shrike_hip_moe *moe, uint32_t num_experts, uint32_t d, uint32_t top_k);
int check_shared(const shrike_projection *gate, const shrike_projection *up, const shrike_projection *down,
                 uint32_t bits, uint32_t d, uint32_t f_shared);

}  // namespace shrike
