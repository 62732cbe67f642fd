// Router logits, top-k select and residency classification for gfx950, and the head
// launch of the fused layer (router rows beside the shared expert's gate/up rows).
#include "decode_launch.h"
#include "rmsnorm_row.h"
#include "router_row.h"

namespace shrike {

// One workgroup's share of MoE.encodeRouter: four expert rows, and the workgroup that finishes last runs
// select (+ classify when a residency table is bound). `tok` picks the token's rows, logits and counter.
template <int RK>
__device__ __forceinline__ void router_block(const RouterArgs &a, size_t tok) {
    __shared__ uint32_t s_last;
    const uint32_t lane = threadIdx.x & 63u, wave = wave_index();
    const uint32_t e = blockIdx.x * 4u + wave;
    const bool select_too = a.lists.out_indices != nullptr;
    // the argument block stays as it is, the token's rows are locals
    const uint16_t *hidden = a.hidden + tok * a.token_stride;
    float *logits = a.logits_out + tok * a.sel.num_experts;
    uint32_t *counter = a.counter + tok;
    if (e < a.sel.num_experts) router_row<RK>(a, hidden, logits, e, lane, select_too);
    if (!select_too) return;  // logits only
    // The logits went out as write-through stores: once they are complete, the workgroup
    // counts itself in; the last to arrive reads all logits back past the caches.
    wait_stores();
    __syncthreads();
    if (threadIdx.x == 0)
        s_last = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == gridDim.x - 1u ? 1u : 0u;
    __syncthreads();
    if (!s_last || wave != 0) return;
    __shared__ RouteScratch s_route;
    SelectArgs sel = a.sel;
    sel.logits = logits;
    RouteLists lists = a.lists;
    lists.out_indices = a.lists.out_indices + tok * a.sel.top_k;
    lists.out_weights = a.lists.out_weights + tok * a.sel.top_k;
    uint32_t cell;
    route_wave<true>(sel, lists, lane, true, cell, s_route);
    if (lane == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// MoE.encodeRouter as one launch; grid.y walks tokens (one in decode).
template <int RK>
__global__ __launch_bounds__(256) void k_router(RouterArgs a) {
    warm_kernel_arguments(a);
    router_block<RK>(a, blockIdx.y);
}

// MoE.encodeRouterPair (router_gemv_r4_pair + router_topk_select_k8_pair, moe.metal:383-408, :511-582): the
// grid's second row is the second router over the same activation row, with logits, counter and outputs of
// its own; the first row is k_router's work exactly.
template <int RK>
__global__ __launch_bounds__(256) void k_router_pair(RouterArgs first, RouterArgs second) {
    if (blockIdx.y == 0) {
        warm_kernel_arguments(first);
        router_block<RK>(first, 0);
    } else {
        warm_kernel_arguments(second);
        router_block<RK>(second, 0);
    }
}

// The head of the fused layer: the router's logit rows and, beside them in the same grid,
// the shared expert's gate and up rows. Neither depends on the other. NORM: every workgroup first
// computes the layer's input row itself (residual add + RMS norm, rmsnorm.metal:96-130) into LDS and
// reads it from there; workgroup 0 also stores it for phase 1.
template <int RK, int BITS, int NCH, bool NORM>
__global__ __launch_bounds__(256) void k_head(RouterArgs r, GemvArgs g, uint32_t router_blocks, NormArgs n) {
    warm_kernel_arguments(r);
    warm_kernel_arguments(g);
    warm_kernel_arguments(n);
    __shared__ uint4 s_x[NORM ? SHRIKE_MAX_HIDDEN / 8 : 1];
    __shared__ float s_partial[4];
    // the norm runs behind the rows' own loads, which do not depend on it
    auto normed_row = [&]() -> const uint4 * {
        rmsnorm_row<false>(const_cast<uint16_t *>(n.hidden), n.delta, n.weight, blockIdx.x == 0 ? n.x_out : nullptr, s_x, r.d, n.eps,
                           s_partial);
        return s_x;
    };
    if (blockIdx.x < router_blocks) {
        const uint32_t e = blockIdx.x * 4u + wave_index();
        // a batch of tokens (no norm, no shared rows): grid.y is the token, with an activation row, a logit row and a
        // route table of its own
        const size_t tok = NORM ? 0u : blockIdx.y;
        if (e < r.sel.num_experts) {
            // what the expert's route entry needs beside the logit: fetched beside the row, used behind it
            const uint16_t bias_bits = r.sel.logit_bias[e], gain_bits = r.sel.per_expert_scale[e];
            const uint64_t word = r.lists.residency ? r.lists.residency[e] : 0;
            float logit;
            if (NORM) logit = router_row<RK>(r, [&] { return reinterpret_cast<const uint16_t *>(normed_row()); }, r.logits_out, e, threadIdx.x & 63u, false);
            else logit = router_row<RK>(r, r.hidden + tok * r.token_stride, r.logits_out + tok * SHRIKE_MAX_ROUTER_EXPERTS, e, threadIdx.x & 63u, false);
            if (r.route_table && (threadIdx.x & 63u) == 0)
                write_route_entry(r.route_table + tok * SHRIKE_MAX_ROUTER_EXPERTS, e, logit, bias_bits, gain_bits, word, r.sel.sigmoid);
        } else if (NORM) {
            normed_row();  // the workgroup's barriers need every wave
        }
    } else {
        if (NORM) gemv_job<BITS, NCH>(g, blockIdx.x - router_blocks, normed_row);
        else gemv_job<BITS, NCH>(g, blockIdx.x - router_blocks);
    }
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
    warm_kernel_arguments(a);
    __shared__ uint32_t s_hit[SHRIKE_MAX_TOP_K], s_miss[SHRIKE_MAX_TOP_K];
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
        s_hit[my_hit_at] = lane;
    } else if (on) {
        a.miss_positions[my_miss_at] = lane;
        a.miss_experts[my_miss_at] = expert;
        a.resolved_slots[lane] = kSentinel;
        s_miss[my_miss_at] = lane;
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
    __syncthreads();
    if (a.tag != 0u && a.host_readback) {
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

int launch_router(const RouterArgs &a, uint32_t router_bits, hipStream_t s) { return launch_router_tokens(a, router_bits, 1, s); }

int launch_router_tokens(const RouterArgs &a, uint32_t router_bits, uint32_t tokens, hipStream_t s) {
    SHRIKE_REQUIRE(tokens == 1 || (a.lists.out_indices && !a.lists.residency), "router: several tokens select only");
    const dim3 grid((a.sel.num_experts + 3) / 4, tokens), block(256);
    if (router_bits == 0) hipLaunchKernelGGL((k_router<0>), grid, block, 0, s, a);
    else if (router_bits == 8) hipLaunchKernelGGL((k_router<8>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((k_router<4>), grid, block, 0, s, a);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

int launch_router_pair(const RouterArgs &first, const RouterArgs &second, uint32_t router_bits, hipStream_t s) {
    const dim3 grid((first.sel.num_experts + 3) / 4, 2), block(256);
    if (router_bits == 0) hipLaunchKernelGGL((k_router_pair<0>), grid, block, 0, s, first, second);
    else if (router_bits == 8) hipLaunchKernelGGL((k_router_pair<8>), grid, block, 0, s, first, second);
    else hipLaunchKernelGGL((k_router_pair<4>), grid, block, 0, s, first, second);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

template <int RK, int BITS>
static void launch_head_nch(const RouterArgs &r, const GemvArgs &g, uint32_t router_blocks, dim3 grid, const NormArgs *norm,
                            hipStream_t s) {
    const dim3 block(256);
    const NormArgs n = norm ? *norm : NormArgs{};
    const uint32_t nch = nch_for(g.n, BITS);
    if (norm) {
        switch (nch) {
            case 1: hipLaunchKernelGGL((k_head<RK, BITS, 1, true>), grid, block, 0, s, r, g, router_blocks, n); break;
            case 2: hipLaunchKernelGGL((k_head<RK, BITS, 2, true>), grid, block, 0, s, r, g, router_blocks, n); break;
            case 3: hipLaunchKernelGGL((k_head<RK, BITS, 3, true>), grid, block, 0, s, r, g, router_blocks, n); break;
            default: hipLaunchKernelGGL((k_head<RK, BITS, 4, true>), grid, block, 0, s, r, g, router_blocks, n); break;
        }
    } else {
        switch (nch) {
            case 1: hipLaunchKernelGGL((k_head<RK, BITS, 1, false>), grid, block, 0, s, r, g, router_blocks, n); break;
            case 2: hipLaunchKernelGGL((k_head<RK, BITS, 2, false>), grid, block, 0, s, r, g, router_blocks, n); break;
            case 3: hipLaunchKernelGGL((k_head<RK, BITS, 3, false>), grid, block, 0, s, r, g, router_blocks, n); break;
            default: hipLaunchKernelGGL((k_head<RK, BITS, 4, false>), grid, block, 0, s, r, g, router_blocks, n); break;
        }
    }
}

// g.rows + g.rows_b == 0: router rows only (g.n must still be a valid row length)
int launch_head(const RouterArgs &r, uint32_t router_bits, const GemvArgs &g, uint32_t shared_bits, const NormArgs *norm,
                hipStream_t s, uint32_t tokens) {
    const uint32_t router_blocks = (r.sel.num_experts + 3) / 4;
    const uint32_t shared_rows = g.rows + g.rows_b;
    SHRIKE_REQUIRE(tokens >= 1 && (tokens == 1 || (shared_rows == 0 && norm == nullptr)), "head launch: a batch of tokens takes router rows only");
    const dim3 grid(router_blocks + (shared_rows ? gemv_blocks(shared_rows, g.n, shared_bits) : 0u), tokens);
    if (shared_bits == 4) {
        if (router_bits == 0) launch_head_nch<0, 4>(r, g, router_blocks, grid, norm, s);
        else if (router_bits == 8) launch_head_nch<8, 4>(r, g, router_blocks, grid, norm, s);
        else launch_head_nch<4, 4>(r, g, router_blocks, grid, norm, s);
    } else {
        if (router_bits == 0) launch_head_nch<0, 8>(r, g, router_blocks, grid, norm, s);
        else if (router_bits == 8) launch_head_nch<8, 8>(r, g, router_blocks, grid, norm, s);
        else launch_head_nch<4, 8>(r, g, router_blocks, grid, norm, s);
    }
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

int check_router(const shrike_hip_moe *moe, uint32_t num_experts, uint32_t d, uint32_t top_k) {
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
    a.d = d; a.meta = moe->desc.meta_dtype;
    a.counter = moe->d_counter; a.logits_out = moe->d_logits;
    a.sel.logits = moe->d_logits;
    a.sel.per_expert_scale = static_cast<const uint16_t *>(d_per_expert_scale);
    a.sel.logit_bias = static_cast<const uint16_t *>(d_logit_bias);
    a.sel.num_experts = num_experts; a.sel.top_k = top_k;
    a.sel.sigmoid = moe->desc.sigmoid_router_scores; a.sel.scaling = moe->desc.routed_scaling_factor;
    a.lists.out_indices = d_out_indices;
    a.lists.out_weights = static_cast<uint16_t *>(d_out_weights);
    return launch_router(a, moe->desc.router_weight_bits, as_stream(stream));
}

const float *shrike_hip_moe_router_logits(const shrike_hip_moe *moe) { return moe ? moe->d_logits : nullptr; }

int shrike_hip_moe_router_pair(shrike_hip_moe *moe, void *stream, const shrike_router_operands *first,
                               const shrike_router_operands *second, const void *d_hidden, const void *d_per_expert_scale,
                               uint32_t num_experts, uint32_t d, uint32_t top_k, float *d_second_logits) {
    SHRIKE_REQUIRE(moe != nullptr, "moe handle is NULL");
    if (int rc = check_router(moe, num_experts, d, top_k)) return rc;
    SHRIKE_REQUIRE(first && second && d_hidden && d_per_expert_scale, "encodeRouterPair: operands, hidden and perExpertScale must be bound");
    const shrike_router_operands *ops[2] = {first, second};
    RouterArgs a[2] = {};
    for (int i = 0; i < 2; ++i) {
        const shrike_router_operands *o = ops[i];
        SHRIKE_REQUIRE(o->weights && o->effective_scale && o->logit_bias, "encodeRouterPair: weights, effectiveScale and logitBias must be bound");
        SHRIKE_REQUIRE(moe->desc.router_weight_bits == 0 || (o->scales && o->biases), "encodeRouterPair: affine router needs scales and biases");
        SHRIKE_REQUIRE(o->out_indices && o->out_weights, "encodeRouterPair: outputs must be bound");
        a[i].weights = o->weights;
        a[i].scales = static_cast<const uint16_t *>(o->scales);
        a[i].biases = static_cast<const uint16_t *>(o->biases);
        a[i].hidden = static_cast<const uint16_t *>(d_hidden);
        a[i].effective_scale = static_cast<const uint16_t *>(o->effective_scale);
        a[i].d = d; a[i].meta = moe->desc.meta_dtype;
        float *logits = i == 0 ? moe->d_logits : (d_second_logits ? d_second_logits : moe->d_logits + SHRIKE_MAX_ROUTER_EXPERTS);
        a[i].counter = moe->d_counter + i; a[i].logits_out = logits;
        a[i].sel.logits = logits;
        a[i].sel.per_expert_scale = static_cast<const uint16_t *>(d_per_expert_scale);
        a[i].sel.logit_bias = static_cast<const uint16_t *>(o->logit_bias);
        a[i].sel.num_experts = num_experts; a[i].sel.top_k = top_k;
        a[i].sel.sigmoid = moe->desc.sigmoid_router_scores; a[i].sel.scaling = moe->desc.routed_scaling_factor;
        a[i].lists.out_indices = o->out_indices;
        a[i].lists.out_weights = static_cast<uint16_t *>(o->out_weights);
    }
    return launch_router_pair(a[0], a[1], moe->desc.router_weight_bits, as_stream(stream));
}

const float *shrike_hip_moe_router_pair_logits(const shrike_hip_moe *moe) {
    return moe ? moe->d_logits + SHRIKE_MAX_ROUTER_EXPERTS : nullptr;
}

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

}  // extern "C"
