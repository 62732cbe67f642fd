/*
 * libshrikehip — the routed-expert (MoE layer) hot path of Shrike on one AMD
 * MI355X (gfx950), behind a plain C ABI in the style of the reference's
 * ShrikeKernelsC target (sources/ShrikeKernelsC/include/shrike_kernels.h).
 *
 * Conventions (the reference's, sources/ShrikeKernelsC/include/shrike_expert_io.h:33-72):
 *  - caller-owned memory; every pointer named `d_*` or documented "device" is a
 *    device address; nothing on a per-layer call allocates;
 *  - every enqueue-only call takes the HIP stream as `void *stream` (a hipStream_t;
 *    NULL = the default stream) and returns at once: ordering is the stream's,
 *    as it is the serial command encoder's in the reference;
 *  - calls return 0 or an errno-style code (EINVAL for what the reference traps
 *    as a precondition, ENOMEM, EIO for a HIP runtime failure);
 *    shrike_hip_last_error() names the cause;
 *  - opaque handles are created with `..._create(..., int *out_errno)` -> NULL on
 *    failure and destroyed with no concurrent callers.
 *
 * Quantised layout (sources/ShrikeKernelsC/include/shrike_kernels.h:11-16,
 * sources/Shrike/Infrastructure/ModelIO/Quantization.swift:30-45): 4-bit codes two
 * per byte, element 2k in the low nibble of byte k; 8-bit codes one per byte; one
 * 16-bit scale and one 16-bit bias per group of 64 along the row, row-major;
 * w = code * scale + bias. The reference stores scale/bias as bf16; fp16 is
 * accepted as well (`meta_dtype`).
 */
#ifndef SHRIKE_HIP_H
#define SHRIKE_HIP_H

#include <stddef.h>
#include <stdint.h>

#include "shrike_host.h"

#ifdef __cplusplus
extern "C" {
#endif

#define SHRIKE_GROUP_SIZE 64u
#define SHRIKE_MAX_TOP_K 8u          /* MoE.maxStreamedExperts, MoE.swift:42 */
#define SHRIKE_MAX_ROUTER_EXPERTS 256u /* MoE.swift:263 */
#define SHRIKE_MAX_HIDDEN 4096u      /* staged activation ceiling (reference: 2880, moe.metal:11) */
#define SHRIKE_POOL_MAX_CHUNKS 8u    /* ExpertCellArena.maxChunks, ExpertCellArena.swift:20 */
#define SHRIKE_SLOT_SENTINEL 0xffffffffu /* ExpertResidencyEntry.notResidentSlot */
#define SHRIKE_POOL_PAGE 16384u      /* .gturbo expert stride alignment, GTurboFormatV1.swift:7 */

enum { SHRIKE_META_BF16 = 0, SHRIKE_META_F16 = 1 };
enum { SHRIKE_ACT_GELU_TANH = 0, SHRIKE_ACT_SILU = 1, SHRIKE_ACT_CLAMPED_SWIGLU = 2 };
enum { SHRIKE_RESIDENCY_EMPTY = 0, SHRIKE_RESIDENCY_LOADING = 1, SHRIKE_RESIDENCY_RESIDENT = 2 };

const char *shrike_hip_last_error(void);
/* 0 when a gfx950 device is present and the kernels' code object loaded. */
int shrike_hip_init(int device);

/* ---------------------------------------------------------------- layouts */

/* shrike_expert_offsets (MoEExpertOffsets) is declared in shrike_host.h. */

/* CPUExpertFFN.Offsets(d:f:), sources/Shrike/Kernels/CPU/CPUExpertFFN.swift:34-61,
 * for 4- or 8-bit codes; additive biases (gpt-oss) are appended when asked for.
 * Returns the packed blob size, 0 on invalid arguments. */
uint64_t shrike_expert_offsets_make(uint32_t d, uint32_t f, uint32_t bits,
                                    int additive_biases, shrike_expert_offsets *out);

/* PoolBases, sources/Shrike/Metal/MoE/moe.metal:297-305: cell -> base[cell /
 * cells_per_chunk] + (cell % cells_per_chunk) * stride. */
typedef struct {
    const void *base[SHRIKE_POOL_MAX_CHUNKS];
    uint32_t cells_per_chunk;
} shrike_pool_bases;

/* SharedExpertProjection, sources/Shrike/Kernels/MoE/SharedExpertInt8.swift:9-31:
 * one resident projection as three device tensors. */
typedef struct {
    const void *weights, *scales, *biases;
} shrike_projection;

/* ------------------------------------------------------ budget -> slot count */

/* RuntimeConfiguration.parseBudgetBytes, sources/Shrike/Runtime/Configuration/
 * RuntimeConfiguration.swift:111-129. Returns bytes, or -1 for what the reference
 * maps to nil. */
int64_t shrike_parse_budget_bytes(const char *text);
/* RuntimeConfiguration.expertCacheSlots, RuntimeConfiguration.swift:77,:137-149. */
int32_t shrike_expert_cache_slots(uint64_t expert_stride_bytes, int32_t layers,
                                  int64_t budget_bytes);

/* ------------------------------------------------------------ HBM slot pool */

/* ExpertCellArena + the residency table of PreadExpertStreamer
 * (sources/Shrike/Infrastructure/Streaming/ExpertCellArena.swift:16-133,
 * PreadExpertStreamer.swift:283-352): `cells` cells of page-rounded stride in at
 * most 8 device chunks, and one 64-bit residency word per expert in device memory
 * (state << 32 | cell). */
typedef struct shrike_hip_pool shrike_hip_pool;
shrike_hip_pool *shrike_hip_pool_create(uint32_t cells, uint64_t expert_stride,
                                        uint32_t num_experts, uint64_t chunk_bytes,
                                        int *out_errno);
/* Another layer's residency table over the same cells: the arena is one for the model
 * (ExpertCellArena.swift:3-8), every layer's streamer owns a range of its cells and a
 * table of its own (PreadExpertStreamer.swift:309-352). The view shares the arena
 * pool's cells and bases, must be destroyed before it, and takes every call a pool takes. */
shrike_hip_pool *shrike_hip_pool_create_layer_view(const shrike_hip_pool *arena,
                                                   uint32_t num_experts, int *out_errno);
void shrike_hip_pool_destroy(shrike_hip_pool *pool);
uint64_t shrike_hip_pool_slot_stride(const shrike_hip_pool *pool);
uint32_t shrike_hip_pool_cell_count(const shrike_hip_pool *pool);
void *shrike_hip_pool_cell_ptr(const shrike_hip_pool *pool, uint32_t cell);
const shrike_pool_bases *shrike_hip_pool_bases(const shrike_hip_pool *pool);
/* device address of the u64[num_experts] residency table */
void *shrike_hip_pool_residency_table(const shrike_hip_pool *pool);
/* Copies one expert blob from host memory (pinned for a truly asynchronous copy)
 * into a cell on `stream`; replaces the reader's pread into the slot
 * (PreadExpertStreamer.swift:610-621). */
int shrike_hip_pool_upload_async(shrike_hip_pool *pool, uint32_t cell, const void *host_src,
                                 uint64_t bytes, void *stream);
/* PreadExpertStreamer.publish, PreadExpertStreamer.swift:1143-1148: stream-ordered
 * store of the expert's residency word; `cell` is ignored for EMPTY. The host
 * shadow is updated at once. */
int shrike_hip_pool_table_publish(shrike_hip_pool *pool, uint32_t expert, uint32_t cell,
                                  uint32_t state, void *stream);
uint64_t shrike_hip_pool_table_entry(const shrike_hip_pool *pool, uint32_t expert);

/* PreadExpertStreamer.executeExpertCachePlan (PreadExpertStreamer.swift:545-574) with the
 * file reads replaced by host-to-device copies: for every miss of `plan` (made by
 * shrike_slot_cache_plan on a cache whose cells are this pool's), expert e is copied from
 * host_store + e * store_expert_stride (pinned memory for an asynchronous copy) into its
 * reserved cell on `stream`; the misses become resident in the cache and every residency
 * word that changed is stored to the device table on the same stream, behind the copies.
 * With two misses or more every other copy runs on a stream of the pool's own, which starts
 * behind everything `stream` holds at the call and which `stream` waits for before the table
 * stores: to the caller the copies are ordered as if all were on `stream` (a stream under
 * capture gets them all itself).
 * The caller orders `stream` against the kernels that still read an evicted cell. */
int shrike_hip_pool_execute_plan(shrike_hip_pool *pool, shrike_slot_cache *cache,
                                 const shrike_expert_cache_plan *plan, const void *host_store, uint64_t store_expert_stride,
                                 uint64_t expert_bytes, void *stream, uint64_t elapsed_nanos);

/* The streamer's read into the slots (PreadExpertStreamer.swift:577-628) for a pool in HBM:
 * `count` blobs of blob_bytes at file_offsets[i] of the reader's layer file (blob_bytes is the
 * stride the reader was created with) are read through the parallel reader into the pinned
 * staging buffer and copied from there into cells[i] on `stream`. The staging buffer is used
 * as two halves, so the reads of one batch run beside the copies of the one before; it must
 * hold at least two blobs. Blocks until the last copy has finished; returns the reader's errno
 * on a failed read (cells already written are then undefined, as the reference's are). */
int shrike_hip_pool_fetch_experts(shrike_hip_pool *pool, void *stream, shrike_expert_reader *reader,
                                  const uint64_t *file_offsets, const uint32_t *cells, uint32_t count,
                                  uint64_t blob_bytes, void *pinned_staging, uint64_t staging_bytes);


/* ------------------------------------------------------------ MoE operators */

/* MoE.init, sources/Shrike/Kernels/MoE/MoE.swift:94-216.
 * Sizes the decode operators take (anything else is EINVAL with a message, never a launch): d and f multiples of 64,
 * d <= SHRIKE_MAX_HIDDEN, and a row of f codes at most 4,096 bytes (f <= 8,192 at 4 bits, f <= 4,096 at 8 bits);
 * num_experts <= SHRIKE_MAX_ROUTER_EXPERTS, top_k <= SHRIKE_MAX_TOP_K. */
typedef struct {
    uint32_t d, f, num_experts, top_k;
    uint32_t routed_weight_bits;   /* 4 | 8 */
    uint32_t router_weight_bits;   /* 0 = fp16 rows, 4 | 8 = group-affine */
    uint32_t meta_dtype;           /* SHRIKE_META_* for every scale/bias tensor */
    uint32_t activation;           /* SHRIKE_ACT_* */
    uint32_t expert_additive_biases;
    uint32_t sigmoid_router_scores;
    float routed_scaling_factor;
    uint32_t event_gated_io;       /* moe.metal:36-39: honour io_status words */
} shrike_moe_desc;

typedef struct shrike_hip_moe shrike_hip_moe;
shrike_hip_moe *shrike_hip_moe_create(const shrike_moe_desc *desc, int *out_errno);
void shrike_hip_moe_destroy(shrike_hip_moe *moe);

/* MoE.encodeRouter, MoE.swift:249-316 (router_gemv_r4 + router_topk_select*,
 * moe.metal:324-381, :419-582). hidden: fp16[d]; effective_scale: bf16[d];
 * per_expert_scale, logit_bias: bf16[num_experts] (always read); out_indices:
 * u32[top_k]; out_weights: fp16[top_k]. Router weights are fp16[num_experts, d]
 * when router_weight_bits == 0 (scales/biases ignored). The fp32 logits land in
 * the handle's own buffer (shrike_hip_moe_router_logits). */
int shrike_hip_moe_router(shrike_hip_moe *moe, void *stream, const void *d_weights,
                          const void *d_scales, const void *d_biases, const void *d_hidden,
                          const void *d_effective_scale, const void *d_per_expert_scale,
                          const void *d_logit_bias, uint32_t *d_out_indices,
                          void *d_out_weights, uint32_t num_experts, uint32_t d,
                          uint32_t top_k);
const float *shrike_hip_moe_router_logits(const shrike_hip_moe *moe);

/* MoE.RouterOperands + MoE.encodeRouterPair, MoE.swift:403-459 (router_gemv_r4_pair and
 * router_topk_select_k8_pair, moe.metal:383-408, :511-582; called at RealForwardRunner.swift:2861):
 * this layer's router and a second one (the next layer's, as the prefetch probe) over the same
 * activation row in one launch. The first router's logits, indices and weights are bit for bit
 * shrike_hip_moe_router's. The second router's fp32 logits go to d_second_logits
 * (fp32[num_experts], the reference's routerLogitsPair at its probe slot) or, when that is NULL,
 * to the handle's own second buffer (shrike_hip_moe_router_pair_logits). */
typedef struct {
    const void *weights, *scales, *biases;      /* as for shrike_hip_moe_router */
    const void *effective_scale, *logit_bias;   /* bf16[d], bf16[num_experts] */
    uint32_t *out_indices;                      /* u32[top_k] */
    void *out_weights;                          /* fp16[top_k] */
} shrike_router_operands;
int shrike_hip_moe_router_pair(shrike_hip_moe *moe, void *stream, const shrike_router_operands *first,
                               const shrike_router_operands *second, const void *d_hidden,
                               const void *d_per_expert_scale, uint32_t num_experts, uint32_t d,
                               uint32_t top_k, float *d_second_logits);
const float *shrike_hip_moe_router_pair_logits(const shrike_hip_moe *moe);

/* MoE.encodeResidencyClassification, MoE.swift:552-610
 * (moe_classify_expert_residency_spec, moe.metal:194-231). `full_grids` are the
 * four full grids (12 words); d_spec_args receives the 12 published words: HIP
 * has no indirect dispatch, so phase1/phase2 below read their grid word from it
 * and return at once when it is zero. d_host_readback (2 + 5*top_k words, may be
 * host-mapped pinned memory) is written when tag != 0. */
int shrike_hip_moe_classify(shrike_hip_moe *moe, void *stream, const uint32_t *d_topk_indices,
                            const uint64_t *d_residency, uint32_t *d_hit_count,
                            uint32_t *d_hit_positions, uint32_t *d_miss_count,
                            uint32_t *d_miss_positions, uint32_t *d_miss_experts,
                            uint32_t *d_resolved_slots, uint32_t top_k, uint32_t num_experts,
                            const uint32_t full_grids[12], uint32_t *d_spec_args,
                            uint32_t *d_host_readback, uint32_t host_readback_tag,
                            const void *d_topk_weights, const uint32_t *d_predicted_indices);

/* MoE.encodeSpecPhase1U16Load, MoE.swift:906-951 (moe_phase1_gate_up_act_spec_u16load,
 * moe.metal:950-999; 8-bit body moe.metal:650-672). x: fp16[d]; acts: fp16[top_k*f].
 * A sentinel in d_resolved_slots skips that position. d_indirect (may be NULL) points
 * at a 3-word grid; a zero first word dispatches nothing. d_io_status may be NULL. */
int shrike_hip_moe_phase1_pool(shrike_hip_moe *moe, void *stream, const shrike_pool_bases *pool,
                               uint64_t pool_slot_stride, const uint32_t *d_resolved_slots,
                               const shrike_expert_offsets *offsets, const void *d_x,
                               void *d_acts, uint32_t d, uint32_t f, uint32_t top_k,
                               const uint32_t *d_indirect, const uint32_t *d_io_status);

/* Argument-buffer addressing: MoE.makeReusedRoutedArgumentBuffer (MoE.swift:612-620) gives position k of the route the
 * blob routedBlobs[k] instead of a pool cell. Here the argument buffer is a device array of top_k pointers
 * (d_routed_blobs[k] = the 16-byte aligned blob of position k; a NULL entry skips the position), which the host
 * fills with an ordinary copy.
 *
 * MoE.encodeRoutedPersistentPhase1U16Load, MoE.swift:651-692 (moe_phase1_gate_up_act_u16load, moe.metal:779-830), and,
 * with d_active_slots bound, MoE.encodeRoutedPersistentPhase1SubsetU16Load, MoE.swift:694-776
 * (moe_phase1_gate_up_act_subset_u16load, moe.metal:832-884): only the positions d_active_slots[0 .. active_count) are
 * computed (an entry >= top_k is skipped), the other positions' acts stay as they are; active_count == 0 with a list
 * bound does nothing. acts: fp16[top_k * f]. */
int shrike_hip_moe_phase1_blobs(shrike_hip_moe *moe, void *stream, const void *const *d_routed_blobs,
                                const shrike_expert_offsets *offsets, const void *d_x, void *d_acts,
                                uint32_t d, uint32_t f, uint32_t top_k, const uint32_t *d_active_slots,
                                uint32_t active_count, const uint32_t *d_io_status);
/* MoE.encodeRoutedPersistentPhase2Reduce, MoE.swift:778-864 (moe_phase2_down_reduce_k8, moe.metal:897-941):
 * shrike_hip_moe_phase2_pool's arithmetic over the argument buffer's blobs. */
int shrike_hip_moe_phase2_blobs(shrike_hip_moe *moe, void *stream, const void *const *d_routed_blobs,
                                const shrike_expert_offsets *offsets, const void *d_acts,
                                const void *d_routing_weights, const void *d_residual, void *d_y,
                                void *d_hidden, uint32_t d, uint32_t f, uint32_t top_k,
                                const uint32_t *d_io_status);

/* MoE.encodeSpecPhase2Reduce, MoE.swift:992-1047 (moe_phase2_down_reduce_spec_k8,
 * moe.metal:1008-1057): y = half(residual + sum_k half_w[k] * down_k . acts_k),
 * hidden = half(hidden + y). A sentinel position takes d_fallback_cells[k] when that
 * is given and contributes nothing otherwise. When event-gated and the status word
 * is not ready, y = residual (moe.metal:918-921). */
int shrike_hip_moe_phase2_pool(shrike_hip_moe *moe, void *stream, const shrike_pool_bases *pool,
                               uint64_t pool_slot_stride, const uint32_t *d_resolved_slots,
                               const uint32_t *d_fallback_cells,
                               const shrike_expert_offsets *offsets, const void *d_acts,
                               const void *d_routing_weights, const void *d_residual,
                               void *d_y, void *d_hidden, uint32_t d, uint32_t f,
                               uint32_t top_k, const uint32_t *d_indirect,
                               const uint32_t *d_io_status);

/* The same operators for a batch of independent decode tokens (several sequences, one token
 * each; RealForwardRunner's batched decode encodes the per-token kernels back to back, here
 * grid.y walks the tokens). resolve: moe.metal:121-151 per position, resolved[t*top_k + p] =
 * cell or SHRIKE_SLOT_SENTINEL, misses added to *d_miss_count when given. phase 1: x is
 * fp16[tokens, x_stride_elements], acts fp16[tokens, top_k, f]. phase 2: routing weights
 * fp16[tokens, top_k]; residual (may be NULL = 0), y and hidden (may be NULL) are
 * fp16[tokens, d]. Per token the results are those of the single-token calls, bit for bit. */
int shrike_hip_moe_resolve_batch(void *stream, const uint32_t *d_topk_indices,
                                 const uint64_t *d_residency, uint32_t *d_resolved_slots,
                                 uint32_t count, uint32_t num_experts, uint32_t *d_miss_count);
int shrike_hip_moe_phase1_batch(shrike_hip_moe *moe, void *stream, const shrike_pool_bases *pool,
                                uint64_t pool_slot_stride, const uint32_t *d_resolved_slots,
                                const shrike_expert_offsets *offsets, const void *d_x,
                                uint32_t x_stride_elements, void *d_acts, uint32_t d, uint32_t f,
                                uint32_t top_k, uint32_t tokens);
int shrike_hip_moe_phase2_batch(shrike_hip_moe *moe, void *stream, const shrike_pool_bases *pool,
                                uint64_t pool_slot_stride, const uint32_t *d_resolved_slots,
                                const shrike_expert_offsets *offsets, const void *d_acts,
                                const void *d_routing_weights, const void *d_residual, void *d_y,
                                void *d_hidden, uint32_t d, uint32_t f, uint32_t top_k,
                                uint32_t tokens);

/* SharedExpertInt4.encodeGateUp + encodeFusedDown / SharedExpertInt8
 * (sources/Shrike/Kernels/MoE/SharedExpertInt4.swift:91-164, :251-342;
 * dequant_int4.metal:206-331, dequant_int8.metal:109-164): h1 = half(down .
 * half(glu(half(gate.x), half(up.x)))), optionally * sigmoid(scalar_gate[0]).
 * d_scratch: fp16[2*f_shared] for the gate and up rows. */
int shrike_hip_shared_expert(shrike_hip_moe *moe, void *stream, const shrike_projection *gate,
                             const shrike_projection *up, const shrike_projection *down,
                             uint32_t bits, const void *d_x, void *d_scratch, void *d_h1,
                             const void *d_scalar_gate, uint32_t d, uint32_t f_shared);

/* The whole decode layer as the runner encodes it
 * (sources/Shrike/Runtime/Inference/RealForwardRunner.swift:2834-2901, :5520-5560):
 * router -> select -> classify -> shared expert -> phase 1 -> phase 2 (+= hidden),
 * in three launches. Same results as the calls above made one after another. */
typedef struct {
    /* router */
    const void *router_weights, *router_scales, *router_biases;
    const void *effective_scale, *per_expert_scale, *logit_bias;
    /* pool */
    const shrike_pool_bases *pool;
    uint64_t pool_slot_stride;
    const uint64_t *residency;
    shrike_expert_offsets offsets;
    /* shared expert (gate.weights == NULL: none, residual = 0) */
    shrike_projection shared_gate, shared_up, shared_down;
    uint32_t shared_bits, shared_f;
    const void *shared_scalar_gate;
    /* activations and outputs */
    const void *x;          /* fp16[d] */
    void *hidden;           /* fp16[d], += y */
    void *y;                /* fp16[d] */
    /* scratch the operator signatures assume (RealForwardRunner.swift:754-825) */
    uint32_t *out_indices;  /* u32[top_k] */
    void *out_weights;      /* fp16[top_k] */
    uint32_t *resolved_slots, *hit_count, *hit_positions, *miss_count, *miss_positions,
        *miss_experts;      /* u32[top_k] / u32[1] */
    void *acts;             /* fp16[top_k*f] */
    void *shared_scratch;   /* fp16[2*shared_f] */
    void *h1;               /* fp16[d] */
    /* the step ahead of the layer fused into its first launch (residual_add_rmsnorm_bf16w,
     * RealForwardRunner.swift:2852-2858, rmsnorm.metal:96-130): with norm_weight != NULL,
     * x = half(half(hidden + norm_delta) * inv * norm_weight) is computed by the call and WRITTEN
     * to x, and hidden ends as half(half(hidden + norm_delta) + y). norm_delta may be NULL (no add).
     * Same bits as shrike_hip_residual_add_rmsnorm_bf16w followed by the layer without these fields. */
    const void *norm_delta;   /* fp16[d] or NULL */
    const void *norm_weight;  /* bf16[d] or NULL: no fused norm */
    float norm_eps;
} shrike_decode_layer_args;
int shrike_hip_moe_decode_layer(shrike_hip_moe *moe, void *stream,
                                const shrike_decode_layer_args *args);
/* The same layer one launch (or any subset) at a time, for a host that encodes other work between them, as
 * the reference's runner does between the shared-expert work, phase 1 and phase 2
 * (RealForwardRunner.swift:5436-5560): `launches` is a mask, bit 0 = router logit rows, route entries and
 * the shared expert's gate/up rows; bit 1 = select + classify, the routed gate/up rows and the shared
 * expert's down rows; bit 2 = the routed down rows, the weighted combine and hidden += y. 7 is
 * shrike_hip_moe_decode_layer. Launches of one layer must run in this order on one stream with the same
 * handle and args, and no other layer call on the handle between them (the route entries live in it). */
int shrike_hip_moe_decode_layer_launches(shrike_hip_moe *moe, void *stream,
                                         const shrike_decode_layer_args *args, uint32_t launches);
/* The same three launches for several sequences that decode one token each (1...16): the runner's layer
 * (RealForwardRunner.swift:2834-2901, :5520-5560) once per sequence, with the token on the grid instead of one call a
 * sequence, so that a batch costs three launches and an expert two sequences route to is found in the caches by the
 * second. Token t reads x + t * x_stride_elements and writes row t of y and hidden (d apart), of out_indices,
 * out_weights and resolved_slots (top_k apart) and of acts (top_k * f apart); per token the bytes are those of
 * shrike_hip_moe_decode_layer. The shared expert and the fused norm must not be bound (they take one token: run
 * shrike_hip_prefill_shared_expert beside this call); the hit and miss lists are not written and may be NULL. */
int shrike_hip_moe_decode_layer_batch(shrike_hip_moe *moe, void *stream, const shrike_decode_layer_args *args,
                                      uint32_t tokens, uint32_t x_stride_elements);

/* The decode layer for callers that cannot allocate (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc). NO COUNTERPART IN THE REFERENCE. Same kernels and same
 * results as shrike_hip_moe_decode_layer, but no handle (shrike_hip_moe_create allocates): the
 * description is passed by value, and the router logits, the route lists, the activations and the
 * shared expert's intermediate rows live in a 96 KiB static device array that each GPU the library
 * runs on holds until the process ends. In `args` the caller binds the inputs (router, pool,
 * residency, shared projections, x, hidden) and the outputs (y, hidden, out_indices, out_weights);
 * the scratch fields (resolved_slots, hit_*, miss_*, acts, shared_scratch, h1) may be NULL and then
 * come from the static array (a caller that reads the miss lists binds those). Limits: f <= 4096,
 * shared_f <= 4096, d <= SHRIKE_MAX_HIDDEN; larger sizes are EINVAL. The call allocates nothing and
 * calls no allocating routine once shrike_hip_init() has run on the device (otherwise its first call
 * on a device looks the array's address up, which must not happen under capture). All calls on one
 * GPU share the array: calls that overlap on one GPU (two streams, two threads) race. */
int shrike_hip_moe_decode_layer_noalloc(const shrike_moe_desc *desc, void *stream,
                                        const shrike_decode_layer_args *args);

/* ------------------------------------------------------- prefill operators */

/* PrefillRouter.encodeBlock, sources/Shrike/Kernels/Prefill/MoE/PrefillRouter.swift:75-152
 * (prefill_router_block_tiled, sources/Shrike/Metal/Prefill/prefill.metal:369-563):
 * the router for query_count tokens. hidden: fp16[query_count, hidden_stride_elements]
 * (row t at t * stride); out_indices: u32[query_count * top_k]; out_weights:
 * fp16[query_count * top_k], token-major. Every token's logits and selection are
 * bit-identical to shrike_hip_moe_router on that token alone. d_workspace is
 * caller-owned, 16-byte aligned, shrike_hip_prefill_router_workspace_bytes() long;
 * the fp32 logits [query_count, num_experts] are left at its start. */
size_t shrike_hip_prefill_router_workspace_bytes(uint32_t query_count, uint32_t num_experts,
                                                 uint32_t d);
int shrike_hip_prefill_router(shrike_hip_moe *moe, void *stream, const void *d_weights,
                              const void *d_scales, const void *d_biases, const void *d_hidden,
                              const void *d_effective_scale, const void *d_per_expert_scale,
                              const void *d_logit_bias, uint32_t *d_out_indices,
                              void *d_out_weights, float *d_workspace,
                              uint32_t query_count, uint32_t num_experts, uint32_t d,
                              uint32_t top_k, uint32_t hidden_stride_elements);
/* The same call, which also leaves at the head of d_ffn_workspace (the grouped FFN's workspace for this chunk, 256-byte
 * aligned) what that FFN first derives from `hidden`: per token and group of 64 elements the fp32 sum, as the FFN's own
 * pass forms it bit for bit. The reference has no such pair of calls: its router (PrefillRouter.swift:75-152) and its
 * grouped GEMMs (PrefillGroupedRoutedMoE.swift:925-1126) each read `hidden` for themselves, and so do the two entry
 * points above and below; this one and shrike_hip_prefill_grouped_ffn_presummed let a runner that hands both the same
 * `hidden` read it once (one launch fewer a chunk). Routes and logits are those of shrike_hip_prefill_router. */
int shrike_hip_prefill_router_with_group_sums(shrike_hip_moe *moe, void *stream, const void *d_weights,
                                              const void *d_scales, const void *d_biases, const void *d_hidden,
                                              const void *d_effective_scale, const void *d_per_expert_scale,
                                              const void *d_logit_bias, uint32_t *d_out_indices,
                                              void *d_out_weights, float *d_workspace,
                                              uint32_t query_count, uint32_t num_experts, uint32_t d,
                                              uint32_t top_k, uint32_t hidden_stride_elements,
                                              void *d_ffn_workspace);

/* One 64-row tile of one expert's pairs: the unit the grouped FFN's workgroups take
 * (the device form of PrefillRoutedExpertBlock + rowTileTable,
 * PrefillGroupedRoutedMoE.swift:71-77, :272-283). `cell` is the expert's pool cell,
 * SHRIKE_SLOT_SENTINEL when the residency table does not hold it. */
typedef struct {
    uint32_t cell, pair_start, rows, expert;
} shrike_row_tile;

/* Device outputs of the grouping (PrefillMoEGroupedRoutes,
 * PrefillMoEGrouping.swift:32-50): sorted_pairs are 16-byte PrefillTokenExpertPair
 * records (token, expert, rank, fp16 weight bits); per_expert_offsets is UINT32_MAX
 * where an expert has no pair. row_tiles has room for
 * shrike_hip_group_max_row_tiles() entries; row_tile_count is one word. */
typedef struct {
    void *sorted_pairs;
    uint32_t *per_expert_offsets;
    uint32_t *per_expert_counts;
    shrike_row_tile *row_tiles;
    uint32_t *row_tile_count;
} shrike_hip_grouped_routes;

uint32_t shrike_hip_group_max_row_tiles(uint64_t pair_count, uint32_t num_experts);

/* PrefillMoEGrouping.groupTokenExpertPairs (PrefillMoEGrouping.swift:269-370) on the
 * device, for the router's token-major output: a stable counting sort by expert, so the
 * order is (sort key, expert, token, rank) exactly as the host function's. Experts are
 * laid out by (d_expert_sort_keys[e], e) when keys are given (u64[num_experts]), by id
 * otherwise. d_residency (u64[num_experts], may be NULL) resolves each expert's cell;
 * with NULL the cell is the expert id. num_experts <= 256. */
int shrike_hip_group_pairs(void *stream, const uint32_t *d_indices, const void *d_weights,
                           uint32_t query_count, uint32_t top_k, uint32_t num_experts,
                           const uint64_t *d_expert_sort_keys, const uint64_t *d_residency,
                           const shrike_hip_grouped_routes *out);

/* PrefillGroupedRoutedMoE.encodeGroupedExpertGEMMs (PrefillGroupedRoutedMoE.swift:925-1126;
 * gather, mpp_prefill_affine_grouped_f16 x3, silu_mul_fp16, scatter —
 * sources/Shrike/Metal/TensorCore/tensorops.metal:61-248, prefill.metal:749-790) for all
 * row tiles in two MFMA launches: route_partials[(token * top_k + rank) * d ..] =
 * fp16(down . fp16(glu(gate . x, up . x))) for every pair of a resident expert.
 * hidden: fp16[query_count, hidden_stride_elements]. d_workspace: caller-owned, at least
 * shrike_hip_prefill_ffn_workspace_bytes(). Tiles of absent experts are skipped (their
 * partial rows are left untouched). */
size_t shrike_hip_prefill_ffn_workspace_bytes(uint32_t query_count, uint32_t max_row_tiles,
                                              uint32_t d, uint32_t f);
int shrike_hip_prefill_grouped_ffn(shrike_hip_moe *moe, void *stream, const shrike_pool_bases *pool,
                                   uint64_t pool_slot_stride, const shrike_expert_offsets *offsets,
                                   const shrike_hip_grouped_routes *routes, uint32_t max_row_tiles,
                                   const void *d_hidden, uint32_t hidden_stride_elements,
                                   void *d_route_partials, void *d_workspace, size_t workspace_bytes,
                                   uint32_t query_count, uint32_t d, uint32_t f, uint32_t top_k);
/* shrike_hip_prefill_grouped_ffn for a d_workspace whose head already holds the group sums of these query_count rows of
 * `hidden` (shrike_hip_prefill_router_with_group_sums on the same stream, same hidden, same d): the same bytes out, without
 * the pass over `hidden` that forms them. */
int shrike_hip_prefill_grouped_ffn_presummed(shrike_hip_moe *moe, void *stream, const shrike_pool_bases *pool,
                                             uint64_t pool_slot_stride, const shrike_expert_offsets *offsets,
                                             const shrike_hip_grouped_routes *routes, uint32_t max_row_tiles,
                                             const void *d_hidden, uint32_t hidden_stride_elements,
                                             void *d_route_partials, void *d_workspace, size_t workspace_bytes,
                                             uint32_t query_count, uint32_t d, uint32_t f, uint32_t top_k);

/* PrefillGroupedRoutedMoE.encodeStreamedBatched (PrefillGroupedRoutedMoE.swift:846-922; kernels
 * prefill_moe_affine_gemv_row_dev and its batched phases, prefill.metal:318-363, :647-728): the
 * routed FFN of the sorted pairs [pair_start, pair_start + pair_count) only — one routed tile of
 * a streamed chunk — with the experts' cells read from d_residency as it stands when the launch
 * runs (NULL: the cells recorded at grouping time). Rows of other pairs are left untouched, and
 * so are the rows of experts the table does not hold. The reference walks the range in
 * microbatches of pair_microbatch_rows pairs through a scalar kernel; here the range goes through
 * the grouped MFMA kernels in one pass, and *out_microbatches reports the count the reference
 * returns. A range need not end at an expert's boundary. Arguments otherwise as for
 * shrike_hip_prefill_grouped_ffn; the workspace may be shared between calls on one stream. */
int shrike_hip_prefill_streamed_batched(shrike_hip_moe *moe, void *stream, const shrike_pool_bases *pool,
                                        uint64_t pool_slot_stride, const shrike_expert_offsets *offsets,
                                        const shrike_hip_grouped_routes *routes, uint32_t max_row_tiles,
                                        const uint64_t *d_residency, uint32_t pair_start,
                                        uint32_t pair_count, uint32_t pair_microbatch_rows,
                                        const void *d_hidden, uint32_t hidden_stride_elements,
                                        void *d_route_partials, void *d_workspace, size_t workspace_bytes,
                                        uint32_t query_count, uint32_t d, uint32_t f, uint32_t top_k,
                                        uint32_t *out_microbatches);

/* The shared expert for query_count tokens (RealForwardRunner.swift:4387-4456: the dense
 * int4/int8 QMMs of MPPPrefillInt4QMM + silu_mul_fp16, then encodeSigmoidScalarMulRows) on the
 * grouped kernel: h1[t, :] = half(down . half(glu(half(gate . x_t), half(up . x_t)))) and, when
 * d_scalar_gate is given, h1[t, :] = half(h1[t, :] * sigmoid(scalar_gate[t])) — ONE GATE A TOKEN,
 * fp16[query_count], as shrike_hip_shared_scalar_gate_rows writes them. The roundings are those of
 * shrike_hip_shared_expert, token by token. h1: fp16[query_count, d]. */
size_t shrike_hip_prefill_shared_expert_workspace_bytes(uint32_t query_count, uint32_t d,
                                                        uint32_t f_shared);
int shrike_hip_prefill_shared_expert(shrike_hip_moe *moe, void *stream, const shrike_projection *gate,
                                     const shrike_projection *up, const shrike_projection *down,
                                     uint32_t bits, const void *d_hidden,
                                     uint32_t hidden_stride_elements, void *d_h1,
                                     const void *d_scalar_gate, void *d_workspace,
                                     size_t workspace_bytes, uint32_t query_count, uint32_t d,
                                     uint32_t f_shared);

/* Elementwise.encodeScalarGateRows, sources/Shrike/Kernels/Primitives/Elementwise.swift:140-164
 * (shared_scalar_gate_rows, moe.metal:1154-1193): the shared expert's scalar gate for a block of tokens,
 * gate[t] = half(dequant8(gate_row) . x_t). gate_row is ONE 8-bit group-affine row (u8[d], 16-bit
 * scale and bias per group of 64); x: fp16[rows, x_stride_elements]; d_gate: fp16[rows]. Eight partial
 * sums added in order as in the reference. d must be a multiple of 64 (Elementwise.swift:148). */
int shrike_hip_shared_scalar_gate_rows(void *stream, const shrike_projection *gate_row, uint32_t meta_dtype,
                                       const void *d_x, uint32_t x_stride_elements, void *d_gate,
                                       uint32_t rows, uint32_t d);
/* Elementwise.encodeSigmoidScalarMulRows, Elementwise.swift:120-138 (sigmoid_scalar_mul_rows_fp16,
 * moe.metal:1195-1207): y[t, i] = half(y[t, i] / (1 + exp(-gate[t]))) in place; y: fp16[rows, d]. */
int shrike_hip_sigmoid_scalar_mul_rows(void *stream, void *d_y, const void *d_gate, uint32_t d, uint32_t rows);

/* PrefillMoE.encodeReduceTokenMajor, sources/Shrike/Kernels/Prefill/MoE/PrefillMoE.swift:11-40
 * (prefill_moe_reduce_token_major, prefill.metal:624-645): h2[t, :] =
 * fp16(sum over ranks, in rank order, of weight[t, r] * partial[t, r, :]). */
int shrike_hip_prefill_reduce(void *stream, const void *d_route_partials, const void *d_route_weights,
                              void *d_h2, uint32_t query_count, uint32_t top_k, uint32_t d);
/* residual_add_fp16 (RealForwardRunner.swift:4658-4665): hidden[i] = fp16(hidden[i] + delta[i]). */
int shrike_hip_residual_add_f16(void *stream, void *d_hidden, const void *d_delta, uint64_t count);
/* The producer of the path's input, RMSNorm.encodeResidualAddBF16W / encodeBF16W
 * (residual_add_rmsnorm_bf16w and rmsnorm_bf16w, sources/Shrike/Metal/Primitives/rmsnorm.metal:70-130;
 * called at RealForwardRunner.swift:2852-2858): per row, hidden = fp16(hidden + delta) in place
 * (d_delta NULL: no add), then out = fp16(hidden * rsqrt(mean(hidden^2) + eps) * bf16 weight), the
 * mean in fp32. The decode call is one row; `rows` rows of d elements are done a workgroup each.
 * Bitwise equal to shrike_hip_residual_add_f16 followed by the norm alone, as in the reference. */
int shrike_hip_residual_add_rmsnorm_bf16w(void *stream, void *d_hidden, const void *d_delta,
                                          const void *d_weight, void *d_out, uint32_t d, float eps,
                                          uint32_t rows);

/* ----------------------------------------------------------------- plumbing
 * Device memory, streams, events and graphs for hosts without a HIP binding of
 * their own (the Python tests and benchmark). No counterpart in the reference,
 * where Metal buffers and command queues play this part
 * (sources/Shrike/Infrastructure/Metal/MetalContext.swift). Pointers returned are
 * NULL on failure; int results are 0 or EIO. Streams are created at the default
 * priority. */
void *shrike_hip_malloc(uint64_t bytes);
int shrike_hip_free(void *device_ptr);
void *shrike_hip_host_alloc(uint64_t bytes);            /* pinned host memory */
int shrike_hip_host_free(void *host_ptr);
int shrike_hip_memcpy_h2d(void *dst, const void *src, uint64_t bytes);
int shrike_hip_memcpy_d2h(void *dst, const void *src, uint64_t bytes);
int shrike_hip_memcpy_d2d(void *dst, const void *src, uint64_t bytes);
int shrike_hip_memcpy_h2d_async(void *dst, const void *src, uint64_t bytes, void *stream);
int shrike_hip_memset(void *dst, int value, uint64_t bytes);
int shrike_hip_device_synchronize(void);
int shrike_hip_mem_info(uint64_t *free_bytes, uint64_t *total_bytes);
void *shrike_hip_stream_create(void);
int shrike_hip_stream_destroy(void *stream);
int shrike_hip_stream_synchronize(void *stream);
void *shrike_hip_event_create(void);
int shrike_hip_event_destroy(void *event);
int shrike_hip_event_record(void *event, void *stream);
int shrike_hip_event_synchronize(void *event);
int shrike_hip_stream_wait_event(void *stream, void *event);
int shrike_hip_event_elapsed_ms(void *start, void *stop, float *ms);
int shrike_hip_graph_begin_capture(void *stream);
void *shrike_hip_graph_end_capture(void *stream);       /* -> executable graph */
int shrike_hip_graph_launch(void *graph_exec, void *stream);
int shrike_hip_graph_destroy(void *graph_exec);

#ifdef __cplusplus
}
#endif
#endif
