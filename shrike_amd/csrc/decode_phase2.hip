// Phase 2 of the routed decode layer for gfx950 (down matvec per selected expert, weighted
// combine, residual, hidden += y: moe.metal:889-941, :1008-1057), the dense group-affine
// GEMV of the shared expert, and the fused-layer entry point.
#include <mutex>

#include "decode_launch.h"

namespace shrike {

constexpr uint32_t kPhase2Rows = 8;       // output rows per workgroup
constexpr uint32_t kPhase2RowsBatch = 16;  // the same for a batch of tokens over rows of more than one wave load

// moe.metal:889-893
__device__ __forceinline__ void phase2_finish(uint16_t *y, uint16_t *hidden, uint32_t d, uint16_t value,
                                              uint16_t hidden_old) {
    y[d] = value;
    if (hidden) hidden[d] = f32_to_f16(f16_to_f32(hidden_old) + f16_to_f32(value));
}

// One wave per routed position (blockDim = 64 * top_k); a workgroup owns kPhase2Rows output
// rows. When a down row is shorter than a wave's 1 KiB load, the wave covers 64/cpr rows per
// load and reduces over lane segments. BATCH row groups are in flight per wave.
// STREAM: one token, every down row is read once: non-temporal row loads (see k_phase1).
// ROWS: output rows a workgroup owns. One token takes 8 (at d = 2048 that is one workgroup a compute unit); a batch of
// tokens over long rows takes 16, so that a wave's slice of the activations, fetched once, serves twice the rows.
// TAIL: the rows end in a step of half chunks (load_slice_regs); NCH then counts the whole steps ahead of it.
// META: the type of the scales and biases (SHRIKE_META_*), known to the instance so that a row converts them one way.
template <int BITS, int NCH, int BATCH, bool STREAM, uint32_t ROWS, bool TAIL, int META>
__global__ __launch_bounds__(512) void k_phase2(Phase2Args a) {
    warm_kernel_arguments(a);
    typedef Chunk<BITS> C;
    constexpr uint32_t kPhase2Rows = ROWS;
    __shared__ float partial[SHRIKE_MAX_TOP_K][kPhase2Rows];
    if (a.indirect && a.indirect[0] == 0u) return;
    // a batch of tokens: grid.y is this workgroup's token (the argument block itself stays untouched)
    const size_t tok = blockIdx.y;
    const uint16_t *acts_tok = a.acts + tok * a.top_k * a.f;
    const uint32_t *resolved_tok = a.resolved + tok * a.top_k;
    const uint32_t *fallback_tok = a.fallback ? a.fallback + tok * a.top_k : nullptr;
    const uint16_t *routing_tok = a.routing_w + tok * a.top_k;
    const uint16_t *residual_tok = a.residual ? a.residual + tok * a.d : nullptr;
    uint16_t *y_tok = a.y + tok * a.d;
    uint16_t *hidden_tok = a.hidden ? a.hidden + tok * a.d : nullptr;
    const uint32_t lane = threadIdx.x & 63u, k = wave_index();
    const uint32_t d0 = blockIdx.x * kPhase2Rows;
    // the epilogue's operands do not depend on anything computed here: fetch them first
    const bool finisher = threadIdx.x < kPhase2Rows && d0 + threadIdx.x < a.d;
    uint16_t res_bits = 0, hid_bits = 0;
    if (finisher) {
        if (residual_tok) res_bits = residual_tok[d0 + threadIdx.x];
        if (hidden_tok) hid_bits = hidden_tok[d0 + threadIdx.x];
        // the residual add of a norm fused ahead of the layer (rmsnorm.metal:104-108) lands here
        if (hidden_tok && a.delta)
            hid_bits = f32_to_f16(__fadd_rn(f16_to_f32(hid_bits), f16_to_f32(a.delta[tok * a.d + d0 + threadIdx.x])));
    }
    if (!io_ready(a.io_status)) {  // moe.metal:1032-1035
        if (finisher) phase2_finish(y_tok, hidden_tok, d0 + threadIdx.x, res_bits, hid_bits);
        return;
    }
    const uint32_t cpr = a.f * BITS / 128u, groups = a.f / kGroup, row_bytes = cpr * 16u;
    // (an instance for rows of more than one step a lane never packs rows: its segment is the wave, and the segment sums'
    // selects fold away)
    constexpr bool kWholeWave = NCH >= 2 || TAIL;
    const bool packed = !kWholeWave && cpr < 64u && (64u % cpr) == 0u;
    const uint32_t rpl = packed ? min(64u / cpr, kPhase2Rows) : 1u;  // rows per wave load
    const uint32_t seg = packed ? cpr : 64u;
    const uint32_t sub = packed ? lane / cpr : 0u, col = packed ? lane % cpr : lane;
    const bool lane_on = sub < rpl;
    const bool writer_lane = (lane & (seg - 1u)) == seg - 1u;  // a segment is a power of two lanes: 64, or a divisor of it

    SliceRegs<BITS, NCH, TAIL> xr;
    load_slice_regs<BITS, NCH, TAIL>(xr, reinterpret_cast<const uint4 *>(acts_tok + size_t(k) * a.f), cpr, col, lane_on);
    const float wk = f16_to_f32(routing_tok[k]);
    bool live;
    const uint8_t *base;
    if (a.blobs) {  // moe.metal:924: the blob the argument buffer names for this position
        base = a.blobs[k];
        live = base != nullptr;
    } else {
        uint32_t cell = resolved_tok[k];
        if (cell == kSentinel && fallback_tok) cell = fallback_tok[k];  // moe.metal:1037-1038
        live = cell != kSentinel;
        base = cell_base_uniform(a.pool, live ? cell : 0u, a.stride);
    }
    const uint16_t *s_all = reinterpret_cast<const uint16_t *>(base + a.off.down_s_off);
    const uint16_t *b_all = reinterpret_cast<const uint16_t *>(base + a.off.down_b_off);

    if (live) {
        const uint32_t n_groups = kPhase2Rows / rpl;
        typename C::X x[NCH];
        float xs[NCH];
        TailX xt;
        for (uint32_t g0 = 0; g0 < n_groups; g0 += BATCH) {
            RowRegs<BITS, NCH, TAIL> rows[BATCH];
            uint32_t row[BATCH];
            bool on[BATCH];
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                row[j] = d0 + (g0 + j) * rpl + sub;
                on[j] = lane_on && (g0 + j) < n_groups && row[j] < a.d;
                const uint32_t rr = on[j] ? row[j] : 0u;
                load_row<BITS, NCH, STREAM, TAIL>(rows[j], base + a.off.down_w_off + size_t(rr) * row_bytes,
                                    s_all + size_t(rr) * groups, b_all + size_t(rr) * groups, cpr, col, on[j]);
            }
            if (g0 == 0) unpack_slices<BITS, NCH, TAIL>(xr, x, xs, xt);
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                float v = seg_sum(row_partial<BITS, NCH, TAIL>(rows[j], x, xs, xt, uint32_t(META)), seg);
                const bool writer = on[j] && writer_lane;
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
        float acc = residual_tok ? f16_to_f32(res_bits) : 0.0f;
        for (uint32_t i = 0; i < a.top_k; ++i) acc += partial[i][threadIdx.x];
        phase2_finish(y_tok, hidden_tok, d0 + threadIdx.x, f32_to_f16(acc), hid_bits);
    }
}

template <int BITS, int NCH>
__global__ __launch_bounds__(256) void k_gemv(GemvArgs a) {
    warm_kernel_arguments(a);
    gemv_job<BITS, NCH>(a, blockIdx.x);
}

template <int BITS, int NCH, uint32_t ROWS, bool TAIL, int META>
static void launch_phase2_meta(const Phase2Args &a, dim3 block, hipStream_t s) {
    const dim3 grid((a.d + ROWS - 1) / ROWS, a.tokens ? a.tokens : 1u);
    const uint32_t cpr = a.f * BITS / 128u;
    const uint32_t rpl = (cpr < 64u && 64u % cpr == 0u) ? (64u / cpr < ROWS ? 64u / cpr : ROWS) : 1u;
    const uint32_t n_groups = ROWS / rpl;  // row groups per wave; up to 4 in flight
    if (a.tokens <= 1u) {
        if (n_groups >= 4) hipLaunchKernelGGL((k_phase2<BITS, NCH, 4, true, ROWS, TAIL, META>), grid, block, 0, s, a);
        else if (n_groups == 2) hipLaunchKernelGGL((k_phase2<BITS, NCH, 2, true, ROWS, TAIL, META>), grid, block, 0, s, a);
        else hipLaunchKernelGGL((k_phase2<BITS, NCH, 1, true, ROWS, TAIL, META>), grid, block, 0, s, a);
    } else {
        if (n_groups >= 4) hipLaunchKernelGGL((k_phase2<BITS, NCH, 4, false, ROWS, TAIL, META>), grid, block, 0, s, a);
        else if (n_groups == 2) hipLaunchKernelGGL((k_phase2<BITS, NCH, 2, false, ROWS, TAIL, META>), grid, block, 0, s, a);
        else hipLaunchKernelGGL((k_phase2<BITS, NCH, 1, false, ROWS, TAIL, META>), grid, block, 0, s, a);
    }
}

template <int BITS, int NCH, uint32_t ROWS, bool TAIL>
static void launch_phase2_rows(const Phase2Args &a, dim3 block, hipStream_t s) {
    if (a.meta == SHRIKE_META_F16) launch_phase2_meta<BITS, NCH, ROWS, TAIL, SHRIKE_META_F16>(a, block, s);
    else launch_phase2_meta<BITS, NCH, ROWS, TAIL, SHRIKE_META_BF16>(a, block, s);
}

// (rows of more than one step a lane, whole or half)
template <int BITS, int NCH, bool TAIL>
static void launch_phase2_batch(const Phase2Args &a, dim3 block, hipStream_t s) {
    if ((NCH >= 2 || TAIL) && a.tokens > 1u) launch_phase2_rows<BITS, NCH, kPhase2RowsBatch, TAIL>(a, block, s);
    else launch_phase2_rows<BITS, NCH, kPhase2Rows, TAIL>(a, block, s);
}

template <int BITS>
static void launch_phase2_bits(const Phase2Args &a, hipStream_t s) {
    const dim3 block(64 * a.top_k);
    const uint32_t cpr = a.f * BITS / 128u;
    if (BITS == 4 && half_chunk_tail(cpr, BITS)) {  // whole steps, then the half chunks
        switch (cpr / 64u) {
            case 1: launch_phase2_batch<BITS, 1, BITS == 4>(a, block, s); break;
            case 2: launch_phase2_batch<BITS, 2, BITS == 4>(a, block, s); break;
            default: launch_phase2_batch<BITS, 3, BITS == 4>(a, block, s); break;
        }
        return;
    }
    switch (nch_for(a.f, BITS)) {
        case 1: launch_phase2_batch<BITS, 1, false>(a, block, s); break;
        case 2: launch_phase2_batch<BITS, 2, false>(a, block, s); break;
        case 3: launch_phase2_batch<BITS, 3, false>(a, block, s); break;
        default: launch_phase2_batch<BITS, 4, false>(a, block, s); break;
    }
}

int launch_phase2(const Phase2Args &a, uint32_t bits, hipStream_t s) {
    if (bits == 4) launch_phase2_bits<4>(a, s); else launch_phase2_bits<8>(a, s);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

template <int BITS>
static void launch_gemv_bits(const GemvArgs &a, hipStream_t s) {
    const dim3 grid(gemv_blocks(a.rows + a.rows_b, a.n, BITS)), block(256);
    switch (nch_for(a.n, BITS)) {
        case 1: hipLaunchKernelGGL((k_gemv<BITS, 1>), grid, block, 0, s, a); break;
        case 2: hipLaunchKernelGGL((k_gemv<BITS, 2>), grid, block, 0, s, a); break;
        case 3: hipLaunchKernelGGL((k_gemv<BITS, 3>), grid, block, 0, s, a); break;
        default: hipLaunchKernelGGL((k_gemv<BITS, 4>), grid, block, 0, s, a); break;
    }
}

int launch_gemv(const GemvArgs &a, uint32_t bits, hipStream_t s) {
    if (bits == 4) launch_gemv_bits<4>(a, s); else launch_gemv_bits<8>(a, s);
    SHRIKE_HIP(hipGetLastError());
    return 0;
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

int check_shared(const shrike_projection *gate, const shrike_projection *up, const shrike_projection *down,
                 uint32_t bits, uint32_t d, uint32_t f_shared) {
    SHRIKE_REQUIRE(gate && up && down && gate->weights && up->weights && down->weights && gate->scales && gate->biases
                   && up->scales && up->biases && down->scales && down->biases,
                   "sharedExpert: gate, up and down projections must be bound");
    SHRIKE_REQUIRE(bits == 4 || bits == 8, "sharedExpert: bits=%u not in {4, 8}", bits);
    SHRIKE_REQUIRE(d % SHRIKE_GROUP_SIZE == 0 && f_shared % SHRIKE_GROUP_SIZE == 0 && f_shared > 0,
                   "sharedExpert: d=%u and f=%u must be multiples of %u", d, f_shared, SHRIKE_GROUP_SIZE);
    SHRIKE_REQUIRE(nch_for(d, bits) <= 4 && nch_for(f_shared, bits) <= 4, "sharedExpert: rows too long");
    // the down projection stages half(glu(gate, up)) for the whole row in an LDS array of SHRIKE_MAX_HIDDEN halves
    SHRIKE_REQUIRE(d <= SHRIKE_MAX_HIDDEN && f_shared <= SHRIKE_MAX_HIDDEN,
                   "sharedExpert: d=%u or f=%u exceeds the activation ceiling %u", d, f_shared, SHRIKE_MAX_HIDDEN);
    return 0;
}

// ---- the static scratch of the allocation-free layer entry point
//
// 96 KiB of device memory that every GPU the library runs on holds until the process ends. Layout (bytes):
// fp32 logits[256] at 0; the route lists (resolved cells, hit/miss counts, positions, experts) at 1024;
// fp16 acts[8 * 4096] at 2048; the shared expert's fp16 gate and up rows [2 * 4096] behind them; fp16 h1[4096];
// the route table (16 bytes an expert, 256 experts) last.
constexpr uint32_t kNoAllocMaxF = 4096, kNoAllocMaxSharedF = 4096;
constexpr size_t kScratchLists = 1024, kScratchActs = 2048;
constexpr size_t kScratchShared = kScratchActs + size_t(SHRIKE_MAX_TOP_K) * kNoAllocMaxF * 2u;
constexpr size_t kScratchH1 = kScratchShared + 2u * kNoAllocMaxSharedF * 2u;
constexpr size_t kScratchRoute = kScratchH1 + size_t(SHRIKE_MAX_HIDDEN) * 2u;  // RouteEntry[256]
constexpr size_t kScratchBytes = kScratchRoute + size_t(SHRIKE_MAX_ROUTER_EXPERTS) * sizeof(RouteEntry);
static_assert(kScratchBytes <= 96u * 1024u, "the static scratch is stated as 96 KiB");
static __device__ __align__(256) unsigned char scratch[96u * 1024u];

// In host code `scratch` is only a handle for the symbol; the array's device address differs from GPU to GPU and is
// looked up once per device, with that device current.
constexpr int kMaxDevices = 64;
static unsigned char *g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mutex;

static int layer_scratch(unsigned char **out) {
    int device = -1;
    SHRIKE_HIP(hipGetDevice(&device));
    SHRIKE_REQUIRE(device >= 0 && device < kMaxDevices, "device %d is past the %d this library keeps scratch for", device, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[device]) {
        void *ptr = nullptr;
        SHRIKE_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        SHRIKE_REQUIRE(ptr != nullptr, "the static scratch has no address on device %d", device);
        g_scratch_ptr[device] = static_cast<unsigned char *>(ptr);
    }
    *out = g_scratch_ptr[device];
    return 0;
}

int init_layer_scratch() {
    unsigned char *ptr = nullptr;
    return layer_scratch(&ptr);
}

}  // namespace shrike

using namespace shrike;

extern "C" {

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
    return launch_phase2(a, bits, as_stream(stream));
}

int shrike_hip_moe_phase2_blobs(shrike_hip_moe *moe, void *stream, const void *const *d_routed_blobs,
                                const shrike_expert_offsets *offsets, const void *d_acts, const void *d_routing_weights,
                                const void *d_residual, void *d_y, void *d_hidden, uint32_t d, uint32_t f, uint32_t top_k,
                                const uint32_t *d_io_status) {
    SHRIKE_REQUIRE(moe != nullptr, "moe handle is NULL");
    SHRIKE_REQUIRE(top_k >= 1 && top_k <= SHRIKE_MAX_TOP_K, "phase2: topK=%u not in 1...8", top_k);
    const uint32_t bits = moe->desc.routed_weight_bits;
    if (int rc = check_offsets(offsets, d, f, bits)) return rc;
    SHRIKE_REQUIRE(d_routed_blobs && d_acts && d_routing_weights && d_residual && d_y,
                   "phase2: the argument buffer, acts, routingWeights, residual and y must be bound");
    Phase2Args a = {};
    a.blobs = reinterpret_cast<const uint8_t *const *>(d_routed_blobs);
    a.off = *offsets;
    a.acts = static_cast<const uint16_t *>(d_acts); a.routing_w = static_cast<const uint16_t *>(d_routing_weights);
    a.residual = static_cast<const uint16_t *>(d_residual);
    a.y = static_cast<uint16_t *>(d_y); a.hidden = static_cast<uint16_t *>(d_hidden);
    a.d = d; a.f = f; a.top_k = top_k; a.meta = moe->desc.meta_dtype; a.ebias = moe->desc.expert_additive_biases;
    a.io_status = moe->desc.event_gated_io ? d_io_status : nullptr;
    return launch_phase2(a, bits, as_stream(stream));
}

// moe.metal:121-151 for a batch: position p of token t resolves to its expert's cell or the sentinel
__global__ __launch_bounds__(256) void k_resolve_batch(const uint32_t *indices, const uint64_t *residency, uint32_t *resolved,
                                                       uint32_t count, uint32_t num_experts, uint32_t *miss_count) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    bool miss = false;
    if (i < count) {
        const uint64_t word = residency[min(indices[i], num_experts - 1u)];
        const bool hit = uint32_t(word >> 32) == SHRIKE_RESIDENCY_RESIDENT && uint32_t(word) != kSentinel;
        resolved[i] = hit ? uint32_t(word) : kSentinel;
        miss = !hit;
    }
    if (miss_count) {
        const uint32_t n = __popcll(__ballot(miss));
        if ((threadIdx.x & 63u) == 0u && n) atomicAdd(miss_count, n);
    }
}

int shrike_hip_moe_resolve_batch(void *stream, const uint32_t *d_topk_indices, const uint64_t *d_residency,
                                 uint32_t *d_resolved_slots, uint32_t count, uint32_t num_experts, uint32_t *d_miss_count) {
    SHRIKE_REQUIRE(d_topk_indices && d_residency && d_resolved_slots, "resolve: indices, residency and resolvedSlots must be bound");
    SHRIKE_REQUIRE(num_experts >= 1, "resolve: numExperts must be positive");
    if (count == 0) return 0;
    hipLaunchKernelGGL(k_resolve_batch, dim3((count + 255u) / 256u), dim3(256), 0, as_stream(stream), d_topk_indices, d_residency,
                       d_resolved_slots, count, num_experts, d_miss_count);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

int shrike_hip_moe_phase2_batch(shrike_hip_moe *moe, void *stream, const shrike_pool_bases *pool,
                                uint64_t pool_slot_stride, const uint32_t *d_resolved_slots,
                                const shrike_expert_offsets *offsets, const void *d_acts, const void *d_routing_weights,
                                const void *d_residual, void *d_y, void *d_hidden, uint32_t d, uint32_t f, uint32_t top_k,
                                uint32_t tokens) {
    SHRIKE_REQUIRE(moe != nullptr && pool != nullptr, "moe handle or pool is NULL");
    SHRIKE_REQUIRE(top_k >= 1 && top_k <= SHRIKE_MAX_TOP_K, "phase2: topK=%u not in 1...8", top_k);
    SHRIKE_REQUIRE(tokens >= 1 && tokens <= 65535u, "phase2: %u tokens not in 1...65535", tokens);
    const uint32_t bits = moe->desc.routed_weight_bits;
    if (int rc = check_offsets(offsets, d, f, bits)) return rc;
    SHRIKE_REQUIRE(d_resolved_slots && d_acts && d_routing_weights && d_y, "phase2: resolvedSlots, acts, routingWeights and y must be bound");
    SHRIKE_REQUIRE(pool_slot_stride % 16u == 0, "phase2: pool slot stride must be a multiple of 16");
    Phase2Args a = {};
    fill_pool(a.pool, pool);
    a.stride = pool_slot_stride; a.resolved = d_resolved_slots; a.off = *offsets;
    a.acts = static_cast<const uint16_t *>(d_acts); a.routing_w = static_cast<const uint16_t *>(d_routing_weights);
    a.residual = static_cast<const uint16_t *>(d_residual);
    a.y = static_cast<uint16_t *>(d_y); a.hidden = static_cast<uint16_t *>(d_hidden);
    a.d = d; a.f = f; a.top_k = top_k; a.meta = moe->desc.meta_dtype; a.ebias = moe->desc.expert_additive_biases;
    a.tokens = tokens;
    return launch_phase2(a, bits, as_stream(stream));
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
    if (int rc = launch_gemv(a, bits, as_stream(stream))) return rc;
    GemvArgs b = {};
    fill_gemv_down(b, down, gate_out, up_out, d_h1, d, f_shared, moe->desc.meta_dtype, moe->desc.activation,
                   d_scalar_gate);
    return launch_gemv(b, bits, as_stream(stream));
}

// Three launches: (1) router logit rows + shared gate/up rows; (2) select + classify in the
// prologue of every phase-1 workgroup, the routed gate/up rows, and the shared down rows;
// (3) phase 2 with the shared expert's output as the residual.
static int decode_layer(shrike_hip_moe *moe, void *stream, const shrike_decode_layer_args *g, uint32_t launches, uint32_t tokens,
                        uint32_t x_stride);

int shrike_hip_moe_decode_layer(shrike_hip_moe *moe, void *stream, const shrike_decode_layer_args *g) {
    return decode_layer(moe, stream, g, 7u, 1u, 0u);
}

int shrike_hip_moe_decode_layer_launches(shrike_hip_moe *moe, void *stream, const shrike_decode_layer_args *g,
                                         uint32_t launches) {
    return decode_layer(moe, stream, g, launches, 1u, 0u);
}

// The same three launches for a batch of sequences, one token each: grid.y walks the tokens in every launch. Token t
// reads x + t * x_stride, selects from its own logit row and route table, and writes row t of y, hidden, out_indices,
// out_weights, resolved_slots and acts. No shared expert and no fused norm (those take one token); hit and miss lists are
// not written.
int shrike_hip_moe_decode_layer_batch(shrike_hip_moe *moe, void *stream, const shrike_decode_layer_args *g, uint32_t tokens,
                                      uint32_t x_stride_elements) {
    SHRIKE_REQUIRE(moe != nullptr && g != nullptr, "moe handle or args is NULL");
    SHRIKE_REQUIRE(tokens >= 1 && tokens <= kLayerBatchTokens, "decodeLayerBatch: %u tokens not in 1...%u", tokens, kLayerBatchTokens);
    SHRIKE_REQUIRE(x_stride_elements >= moe->desc.d && x_stride_elements % 8u == 0, "decodeLayerBatch: x stride is too small or leaves rows unaligned");
    SHRIKE_REQUIRE(g->shared_gate.weights == nullptr && g->norm_weight == nullptr,
                   "decodeLayerBatch: the shared expert and the fused norm take one token; run them as operators of their own");
    return decode_layer(moe, stream, g, 7u, tokens, x_stride_elements);
}

static int decode_layer(shrike_hip_moe *moe, void *stream, const shrike_decode_layer_args *g, uint32_t launches, uint32_t tokens,
                        uint32_t x_stride) {
    SHRIKE_REQUIRE(moe != nullptr && g != nullptr, "moe handle or args is NULL");
    const bool batch = tokens > 1u || x_stride != 0u;
    SHRIKE_REQUIRE(launches != 0 && launches <= 7u, "decodeLayer: launches=%u is not a mask of the three launches", launches);
    const shrike_moe_desc &m = moe->desc;
    if (int rc = check_router(moe, m.num_experts, m.d, m.top_k)) return rc;
    if (int rc = check_offsets(&g->offsets, m.d, m.f, m.routed_weight_bits)) return rc;
    SHRIKE_REQUIRE(g->router_weights && g->effective_scale && g->per_expert_scale && g->logit_bias,
                   "decodeLayer: router operands must be bound");
    SHRIKE_REQUIRE(m.router_weight_bits == 0 || (g->router_scales && g->router_biases),
                   "decodeLayer: affine router needs scales and biases");
    SHRIKE_REQUIRE(g->pool && g->residency && g->x && g->y && g->out_indices && g->out_weights && g->resolved_slots && g->acts,
                   "decodeLayer: pool, residency, x, y and the scratch buffers must be bound");
    SHRIKE_REQUIRE(batch || (g->hit_count && g->hit_positions && g->miss_count && g->miss_positions && g->miss_experts),
                   "decodeLayer: pool, residency, x, y and the scratch buffers must be bound");
    SHRIKE_REQUIRE(g->pool_slot_stride % 16u == 0, "decodeLayer: pool slot stride must be a multiple of 16");
    const bool normed = g->norm_weight != nullptr;
    NormArgs norm = {};
    if (normed) {  // x = rmsnorm(hidden + delta) * weight is this call's own first step; x is written
        SHRIKE_REQUIRE(g->hidden, "decodeLayer: a fused norm reads hidden");
        SHRIKE_REQUIRE(m.d % 8u == 0 && m.d <= SHRIKE_MAX_HIDDEN, "decodeLayer: d=%u is not a row the norm takes", m.d);
        SHRIKE_REQUIRE(((reinterpret_cast<uintptr_t>(g->hidden) | reinterpret_cast<uintptr_t>(g->norm_delta)
                         | reinterpret_cast<uintptr_t>(g->norm_weight) | reinterpret_cast<uintptr_t>(g->x)) & 15u) == 0,
                       "decodeLayer: hidden, delta, norm weight and x must be 16-byte aligned");
        norm.hidden = static_cast<const uint16_t *>(g->hidden);
        norm.delta = static_cast<const uint16_t *>(g->norm_delta);
        norm.weight = static_cast<const uint16_t *>(g->norm_weight);
        norm.x_out = static_cast<uint16_t *>(const_cast<void *>(g->x));
        norm.eps = g->norm_eps;
    }
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
    r.sel.logits = moe->d_logits;
    r.sel.per_expert_scale = static_cast<const uint16_t *>(g->per_expert_scale);
    r.sel.logit_bias = static_cast<const uint16_t *>(g->logit_bias);
    r.sel.num_experts = m.num_experts; r.sel.top_k = m.top_k;
    r.sel.sigmoid = m.sigmoid_router_scores; r.sel.scaling = m.routed_scaling_factor;
    // launch 1 writes the logits and, beside each, the expert's route entry; no list yet
    r.lists.residency = g->residency;
    r.route_table = moe->d_route;
    r.token_stride = x_stride;

    Phase1Args p1 = {};
    fill_pool(p1.pool, g->pool);
    p1.stride = g->pool_slot_stride; p1.resolved = g->resolved_slots; p1.off = g->offsets;
    p1.x = static_cast<const uint16_t *>(g->x); p1.acts = static_cast<uint16_t *>(g->acts);
    p1.d = m.d; p1.f = m.f; p1.top_k = m.top_k; p1.meta = m.meta_dtype; p1.act = m.activation;
    p1.ebias = m.expert_additive_biases;
    p1.sel = r.sel;
    p1.lists.out_indices = g->out_indices; p1.lists.out_weights = static_cast<uint16_t *>(g->out_weights);
    p1.lists.residency = g->residency; p1.lists.resolved_slots = g->resolved_slots;
    if (!batch) {  // a batch writes the cells alone
        p1.lists.hit_count = g->hit_count; p1.lists.hit_positions = g->hit_positions;
        p1.lists.miss_count = g->miss_count; p1.lists.miss_positions = g->miss_positions;
        p1.lists.miss_experts = g->miss_experts;
    }
    p1.tokens = tokens; p1.x_stride = x_stride;
    p1.route_table = moe->d_route;
    p1.routed_blocks = phase1_blocks(m.top_k, m.f);

    const void *residual = nullptr;
    bool down_fused = false;
    if (shared) {
        GemvArgs gu = {};
        fill_gemv_gate_up(gu, &g->shared_gate, &g->shared_up, gate_out, up_out, g->shared_f, m.d, m.meta_dtype, g->x);
        if (launches & 1u)
            if (int rc = launch_head(r, m.router_weight_bits, gu, sbits, normed ? &norm : nullptr, s)) return rc;
        fill_gemv_down(p1.shared_down, &g->shared_down, gate_out, up_out, g->h1, m.d, g->shared_f, m.meta_dtype,
                       m.activation, g->shared_scalar_gate);
        down_fused = nch_for(g->shared_f, sbits) == 1;
        residual = g->h1;
    } else {  // the head launch with router rows only
        GemvArgs none = {};
        none.n = m.d;
        if (launches & 1u)
            if (int rc = launch_head(r, m.router_weight_bits, none, sbits, normed ? &norm : nullptr, s, tokens)) return rc;
    }
    if (launches & 2u) {
        if (int rc = launch_phase1(p1, m.routed_weight_bits, true, down_fused ? sbits : 0u, s)) return rc;
        if (shared && !down_fused) {
            if (int rc = launch_gemv(p1.shared_down, sbits, s)) return rc;
        }
    }
    if (!(launches & 4u)) return 0;

    Phase2Args p = {};
    fill_pool(p.pool, g->pool);
    p.stride = g->pool_slot_stride; p.resolved = g->resolved_slots; p.off = g->offsets;
    p.acts = static_cast<const uint16_t *>(g->acts); p.routing_w = static_cast<const uint16_t *>(g->out_weights);
    p.residual = static_cast<const uint16_t *>(residual);
    p.y = static_cast<uint16_t *>(g->y); p.hidden = static_cast<uint16_t *>(g->hidden);
    p.d = m.d; p.f = m.f; p.top_k = m.top_k; p.meta = m.meta_dtype; p.ebias = m.expert_additive_biases;
    p.delta = normed ? norm.delta : nullptr;
    p.tokens = tokens;
    return launch_phase2(p, m.routed_weight_bits, s);
}

// The same layer for callers that cannot allocate: no handle (making one allocates), no scratch from the caller.
// The kernels are the ones above; the logits, the route lists, the activations and the shared expert's
// intermediate rows live in the static array. Calls that overlap on one GPU race on it.
int shrike_hip_moe_decode_layer_noalloc(const shrike_moe_desc *desc, void *stream, const shrike_decode_layer_args *g) {
    if (int rc = check_moe_desc(desc)) return rc;
    SHRIKE_REQUIRE(g != nullptr, "args is NULL");
    SHRIKE_REQUIRE(desc->f <= kNoAllocMaxF, "decodeLayerNoAlloc: f=%u exceeds the static scratch's %u", desc->f, kNoAllocMaxF);
    SHRIKE_REQUIRE(g->shared_gate.weights == nullptr || g->shared_f <= kNoAllocMaxSharedF,
                   "decodeLayerNoAlloc: sharedF=%u exceeds the static scratch's %u", g->shared_f, kNoAllocMaxSharedF);
    if (stream != nullptr) {
        // every GPU holds its own copy of the array: the one used must be the one of the GPU the launches go to
        int current = -1;
        hipDevice_t of_stream = -1;
        SHRIKE_HIP(hipGetDevice(&current));
        SHRIKE_HIP(hipStreamGetDevice(as_stream(stream), &of_stream));
        SHRIKE_REQUIRE(int(of_stream) == current, "decodeLayerNoAlloc: the stream belongs to device %d, the current device is %d",
                       int(of_stream), current);
    }
    unsigned char *base = nullptr;
    if (int rc = layer_scratch(&base)) return rc;
    shrike_hip_moe moe = {};
    moe.desc = *desc;
    moe.d_logits = reinterpret_cast<float *>(base);
    moe.d_counter = nullptr;  // the fused layer selects in the second launch's prologue: no arrival counter
    moe.d_route = reinterpret_cast<RouteEntry *>(base + kScratchRoute);
    shrike_decode_layer_args a = *g;
    uint32_t *lists = reinterpret_cast<uint32_t *>(base + kScratchLists);
    if (!a.resolved_slots) a.resolved_slots = lists;
    if (!a.hit_positions) a.hit_positions = lists + 8;
    if (!a.miss_positions) a.miss_positions = lists + 16;
    if (!a.miss_experts) a.miss_experts = lists + 24;
    if (!a.hit_count) a.hit_count = lists + 32;
    if (!a.miss_count) a.miss_count = lists + 33;
    if (!a.acts) a.acts = base + kScratchActs;
    if (!a.shared_scratch) a.shared_scratch = base + kScratchShared;
    if (!a.h1) a.h1 = base + kScratchH1;
    return shrike_hip_moe_decode_layer(&moe, stream, &a);
}

}  // extern "C"
