/*
 * libshrikehip, host side: the integer bookkeeping around the routed-expert path —
 * token/expert pair records, the grouping permutation, the expert sweep order, the
 * staging-wave planner and the slot cache. Plain C ABI, caller-owned memory, no
 * device calls (the functions here run without a GPU); same conventions as
 * shrike_hip.h. Where the reference throws a Swift error the call returns a
 * nonzero code and shrike_hip_last_error() carries the reference's message.
 */
#ifndef SHRIKE_HOST_H
#define SHRIKE_HOST_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------ pair records */

/* PrefillTokenExpertPair, sources/Shrike/Kernels/Prefill/MoE/PrefillRouter.swift:5-28
 * (16 bytes; the fp16 weight's bits sit in the low half of the fourth word). */
typedef struct {
    uint32_t token, expert, rank, weight_bits_and_reserved;
} shrike_token_expert_pair;

/* PrefillRouter.makeTokenExpertPairs, PrefillRouter.swift:160-180: token-major
 * records from the router's [query_count * top_k] indices and fp16 weights. */
int shrike_make_token_expert_pairs(const uint32_t *indices, const uint16_t *weights_f16,
                                   uint32_t query_count, uint32_t top_k,
                                   shrike_token_expert_pair *out_pairs);

/* ---------------------------------------------------------------- grouping */

/* PrefillMoEGroup / PrefillMoETile, PrefillMoEGrouping.swift:4-30. */
typedef struct {
    uint32_t expert, pair_start, pair_count;
} shrike_moe_group;
typedef struct {
    uint32_t group_start, group_count, pair_start, pair_count;
} shrike_moe_tile;

/* PrefillMoEGroupingError, PrefillMoEGrouping.swift:52-89, in declaration order. */
enum {
    SHRIKE_GROUPING_OK = 0,
    SHRIKE_GROUPING_INVALID_QUERY_COUNT = 1,
    SHRIKE_GROUPING_INVALID_TOP_K = 2,
    SHRIKE_GROUPING_INVALID_NUM_EXPERTS = 3,
    SHRIKE_GROUPING_INVALID_TILE_EXPERT_COUNT = 4,
    SHRIKE_GROUPING_PAIR_COUNT_MISMATCH = 5,
    SHRIKE_GROUPING_TOKEN_OUT_OF_RANGE = 6,
    SHRIKE_GROUPING_RANK_OUT_OF_RANGE = 7,
    SHRIKE_GROUPING_EXPERT_OUT_OF_RANGE = 8,
    SHRIKE_GROUPING_DUPLICATE_TOKEN_RANK = 9,
    SHRIKE_GROUPING_EXPERT_SORT_KEY_COUNT_MISMATCH = 10
};

/* PrefillMoEGroupedRoutes, PrefillMoEGrouping.swift:32-50. The caller provides
 * sorted_pairs[pair_count], per_expert_offsets[num_experts], per_expert_counts
 * [num_experts], groups and tiles [min(num_experts, pair_count)]; the counts and
 * maxima are written by the call. */
typedef struct {
    shrike_token_expert_pair *sorted_pairs;
    uint32_t *per_expert_offsets; /* UINT32_MAX where the expert has no pair */
    uint32_t *per_expert_counts;
    shrike_moe_group *groups;
    shrike_moe_tile *tiles;
    uint32_t group_count, tile_count;
    uint32_t max_pairs_per_expert, max_pairs_per_tile, max_live_experts_per_tile;
    /* the two values of the reference's error case (0 where it has fewer) */
    int64_t error_value[2];
} shrike_grouped_routes;

/* PrefillMoEGrouping.groupTokenExpertPairs, PrefillMoEGrouping.swift:269-370;
 * called at RealForwardRunner.swift:4352. expert_sort_keys may be NULL (then
 * sort_key_count is ignored). Returns a SHRIKE_GROUPING_* code. */
int shrike_group_pairs(const shrike_token_expert_pair *pairs, size_t pair_count,
                       int64_t query_count, int64_t top_k, int64_t num_experts,
                       int64_t tile_expert_count, const uint64_t *expert_sort_keys,
                       size_t sort_key_count, shrike_grouped_routes *out);

/* -------------------------------------------------------------- sweep order */

/* PrefillSweepOrder.residentFirstBalanced, PrefillMoEGrouping.swift:131-177. The
 * chunk's routed experts come as parallel arrays (expert id, rows, last row; ids
 * distinct); resident[e] != 0 marks an expert the pool holds (ids past
 * resident_count count as absent). out_order has room for `count` ids. */
int shrike_sweep_order_resident_first_balanced(const uint32_t *experts, const int64_t *rows,
                                               const int64_t *last_row, size_t count,
                                               const uint8_t *resident, size_t resident_count,
                                               int64_t slots, int64_t tile_width,
                                               uint32_t *out_order, size_t *out_count);

/* PrefillSweepOrder.expertSortKeys, PrefillMoEGrouping.swift:196-202. */
void shrike_expert_sort_keys(const uint32_t *order, size_t count, size_t num_experts,
                             uint64_t *out_keys);

/* -------------------------------------------------------------- wave planner */

/* PrefillExpertPairRange, PrefillGroupedRoutedMoE.swift:33-43. */
typedef struct {
    uint32_t expert;
    int64_t pair_start, pair_count;
} shrike_expert_pair_range;

/* PrefillRoutedExpertBlock, PrefillGroupedRoutedMoE.swift:71-77 (5 x u32, the
 * layout the kernels read). */
typedef struct {
    uint32_t slot, pair_start, rows, staging_row, row_tile_start;
} shrike_routed_expert_block;

/* PrefillRoutedExpertWave, PrefillGroupedRoutedMoE.swift:83-89, with its blocks
 * as a range of the flat block array. */
typedef struct {
    uint32_t block_start, block_count, padded_rows, tail_rows;
} shrike_routed_expert_wave;

/* PrefillGroupedRoutedMoE.planExpertWaves, PrefillGroupedRoutedMoE.swift:104-241;
 * called at RealForwardRunner.swift:4910. An expert's slot is its position in
 * bound_experts (PrefillStreamedTileBinding.localSlot). row_tile 64 (or 32 with
 * tail_tile 0); tail_tile 0 or 32. EINVAL for what the reference throws
 * (staging rows, unbound expert, tile combination), ENOSPC when blocks/waves
 * are too small (the counts needed are still written). */
int shrike_plan_expert_waves(const shrike_expert_pair_range *ranges, size_t range_count,
                             const uint32_t *bound_experts, size_t bound_count,
                             int64_t staging_rows, int64_t row_tile, int64_t tail_tile,
                             shrike_routed_expert_block *blocks, size_t block_capacity,
                             size_t *block_count, shrike_routed_expert_wave *waves,
                             size_t wave_capacity, size_t *wave_count);

/* rowTileTable, PrefillGroupedRoutedMoE.swift:272-283: table[t] = index (within the
 * wave) of the block that owns row tile t; padded_rows / row_tile entries. */
int shrike_row_tile_table(const shrike_routed_expert_block *blocks, size_t block_count,
                          uint32_t padded_rows, uint32_t row_tile, uint32_t *table);

/* rowTileTables, PrefillGroupedRoutedMoE.swift:247-269: gather (padded_rows / 32),
 * body ((padded_rows - tail_rows) / 64) and tail (tail_rows / 32) tables. */
int shrike_row_tile_tables(const shrike_routed_expert_block *blocks, size_t block_count,
                           uint32_t padded_rows, uint32_t tail_rows, uint32_t *gather,
                           uint32_t *body, uint32_t *tail);

/* ---------------------------------------------------------------- slot cache */

/* ExpertCellArena's numbering and generations
 * (sources/Shrike/Infrastructure/Streaming/ExpertCellArena.swift:16-29, :95-104): every
 * cell a residency word can name, the pool slots of every layer and the prefetch ring's
 * cells alike, with one clock behind all generations. The cells' bytes are the HBM
 * pool's; this object holds the numbering only. It must outlive the caches made in it. */
typedef struct shrike_cell_arena shrike_cell_arena;
shrike_cell_arena *shrike_cell_arena_create(uint32_t cell_count, int *out_errno);
void shrike_cell_arena_destroy(shrike_cell_arena *arena);
uint32_t shrike_cell_arena_cell_count(const shrike_cell_arena *arena);
/* cellGeneration, ExpertCellArena.swift:95-98; 0 for a cell outside the arena. */
uint64_t shrike_cell_arena_generation(const shrike_cell_arena *arena, uint32_t cell);

/* The slot bookkeeping of PreadExpertStreamer
 * (sources/Shrike/Infrastructure/Streaming/PreadExpertStreamer.swift:405-543,
 * :676-767, :1085-1148): hit lookup, victim choice, loading/resident states, cell
 * generations, pins, statistics and the residency words; and the landings and overflow
 * slots of :815-1018. One lock guards it, as in the reference. Slot s starts at pool cell
 * first_cell + s; adopting a landing gives the slot the landing's cell. */
typedef struct shrike_slot_cache shrike_slot_cache;

/* ExpertEvictionPolicy, sources/Shrike/Runtime/Inference/Model.swift:22-41. */
enum { SHRIKE_EVICT_AGING_LFU = 0, SHRIKE_EVICT_SLRU = 1 };

/* A cache over an arena of its own, first_cell + slot_count cells long. */
shrike_slot_cache *shrike_slot_cache_create(uint32_t slot_count, uint32_t experts_per_layer,
                                            uint32_t first_cell, int policy,
                                            double slru_protected_share, int *out_errno);
/* PreadExpertStreamer.init(arena:cellRange:), PreadExpertStreamer.swift:309-319: the slots
 * take cells first_cell ..< first_cell + slot_count of a shared arena. */
shrike_slot_cache *shrike_slot_cache_create_in_arena(shrike_cell_arena *arena, uint32_t slot_count,
                                                     uint32_t experts_per_layer, uint32_t first_cell,
                                                     int policy, double slru_protected_share,
                                                     int *out_errno);
void shrike_slot_cache_destroy(shrike_slot_cache *cache);

/* ExpertCachePlan, PreadExpertStreamer.swift:17-38. Arrays are caller-provided with room
 * for expert_count entries; experts is copied in by the plan call. assigned_cells (the
 * arena cell behind each assigned slot) is optional; adopted (indices into experts),
 * freed_experts and freed_cells (freedCells as pairs) are needed only by a plan that is
 * given leased landings, and may be NULL otherwise. */
typedef struct {
    uint32_t expert_count;
    int32_t layer;
    int32_t *experts;
    int32_t *assigned_slots;
    uint64_t *assigned_generations;
    uint32_t *misses; /* indices into experts */
    uint32_t miss_count;
    uint32_t hits;
    uint32_t *assigned_cells;
    uint32_t *adopted;
    uint32_t adopted_count;
    uint32_t freed_count;
    int32_t *freed_experts;
    uint32_t *freed_cells;
} shrike_expert_cache_plan;

/* makeExpertCachePlan, PreadExpertStreamer.swift:405-543 (planExpertsCached /
 * planExpertsCachedIfPossible). avoiding_slots and protected_experts may be NULL;
 * misses_counted < 0 counts the plan's own misses. Returns 0, ENOSPC when the
 * experts cannot be placed (the reference's nil / expertCacheUnplaceable), EINVAL
 * when expert_count exceeds the slot count. */
int shrike_slot_cache_plan(shrike_slot_cache *cache, const int32_t *experts, uint32_t expert_count,
                           int32_t layer, const int32_t *avoiding_slots, uint32_t avoiding_count,
                           const uint8_t *protected_experts, uint32_t protected_count,
                           int64_t misses_counted, shrike_expert_cache_plan *plan);
/* The same with gpuMissedExperts and leasedLandings (:499-515): a miss whose expert has a
 * completed landing leased to the plan takes the landing's cell as its slot's cell and is
 * a hit of the plan; the slot's former cell is reported in freed_cells for the ring to
 * reuse, and the index is listed in adopted when the GPU had missed the expert. */
int shrike_slot_cache_plan_with_landings(shrike_slot_cache *cache, const int32_t *experts,
                                         uint32_t expert_count, int32_t layer,
                                         const int32_t *avoiding_slots, uint32_t avoiding_count,
                                         const uint8_t *protected_experts, uint32_t protected_count,
                                         const int32_t *gpu_missed_experts, uint32_t gpu_missed_count,
                                         const int32_t *leased_landings, uint32_t leased_count,
                                         int64_t misses_counted, shrike_expert_cache_plan *plan);
/* markPlanMissesResident + the success leg of finishPlanExecution
 * (PreadExpertStreamer.swift:1085-1105, :1070-1083): the plan's misses become
 * resident and are counted as one load batch. EIO when a generation changed. */
int shrike_slot_cache_complete(shrike_slot_cache *cache, const shrike_expert_cache_plan *plan,
                               uint64_t elapsed_nanos, uint64_t fetch_nanos);
/* abandonExpertCachePlan, PreadExpertStreamer.swift:1110-1128. */
void shrike_slot_cache_abandon(shrike_slot_cache *cache, const shrike_expert_cache_plan *plan);
/* pin / unpin, PreadExpertStreamer.swift:744-778. pin returns EIO on a stale plan. */
int shrike_slot_cache_pin(shrike_slot_cache *cache, const shrike_expert_cache_plan *plan);
void shrike_slot_cache_unpin(shrike_slot_cache *cache, const int32_t *slots,
                             const uint64_t *generations, uint32_t count);

/* cellIndexUnlocked, PreadExpertStreamer.swift:1135-1137: the arena cell behind a slot
 * (-1 for a slot out of range), and ownsCell, :1021-1025. */
int64_t shrike_slot_cache_slot_cell(shrike_slot_cache *cache, uint32_t slot);
int shrike_slot_cache_owns_cell(shrike_slot_cache *cache, uint32_t cell);

/* claimLanding, PreadExpertStreamer.swift:815-829: a ring cell claimed for a prediction's
 * read, `loading` for the classifier and neither a hit nor a victim for a plan. 1 when
 * claimed; 0 when the pool holds or is loading the expert, a landing for it exists,
 * another landing holds the cell, or an argument is out of range. */
int shrike_slot_cache_claim_landing(shrike_slot_cache *cache, int32_t expert, int64_t cell);
/* completeLanding, :834-848: `resident` at the cell; 0 (nothing published) for a landing
 * that was dropped, re-claimed, or overtaken by the pool's own read of the expert. */
int shrike_slot_cache_complete_landing(shrike_slot_cache *cache, int32_t expert, int64_t cell);
/* failLanding / dropLanding, :850-852, :1010-1018: the entry is emptied unless the pool
 * owns the expert. */
void shrike_slot_cache_fail_landing(shrike_slot_cache *cache, int32_t expert, int64_t cell);
void shrike_slot_cache_drop_landing(shrike_slot_cache *cache, int32_t expert, int64_t cell);
/* The claims of beginPrefetch, :1034-1057: every cell must be outside the pool (EINVAL,
 * like an expert out of range); a refused claim drops the batch's earlier ones, stores
 * its index and returns SHRIKE_PREFETCH_CLAIM_REFUSED. The caller issues the reads and
 * reports each landing with complete_landing or fail_landing. */
int shrike_slot_cache_claim_prefetch(shrike_slot_cache *cache, const int32_t *experts,
                                     const int64_t *cells, uint32_t count, uint32_t *refused_index);

/* reserveOverflowSlot, :860-893: a pool slot for a miss the ring could not house: the
 * policy's victim among the slots not holding `protecting`, evicted and `loading` at its
 * cell, on probation for SLRU. Returns the cell, or -1 when no slot is evictable or the
 * pool already holds the expert. */
int64_t shrike_slot_cache_reserve_overflow_slot(shrike_slot_cache *cache, int32_t expert,
                                                const int32_t *protecting, uint32_t protecting_count);
/* markOverflowResident, :968-976, and abandonOverflowSlot / emptyOverflowSlot, :980-993. */
void shrike_slot_cache_mark_overflow_resident(shrike_slot_cache *cache, int32_t expert, int64_t cell);
void shrike_slot_cache_abandon_overflow_slot(shrike_slot_cache *cache, int32_t expert, int64_t cell);
/* The completion leg of beginAgreedReads, :936-964, :995-1002: on success every pool cell
 * turns resident and every ring cell's landing completes, and the batch is counted; on
 * failure the landings are dropped and the pool cells emptied. */
int shrike_slot_cache_finish_agreed_reads(shrike_slot_cache *cache, const int32_t *experts,
                                          const int64_t *cells, uint32_t count, int succeeded,
                                          uint64_t elapsed_nanos, uint64_t fetch_nanos);

/* ExpertStreamingStatistics, PreadExpertStreamer.swift:40-71 (the fields this
 * library maintains). */
typedef struct {
    uint64_t plans, requested_experts, hits, misses, bytes_read, read_operations;
    uint64_t evictions, reloads, load_batches, total_load_nanos, fetch_nanos, maximum_load_nanos;
    uint64_t latency_histogram[17];
    uint32_t resident_slots, loading_slots, pinned_slots, peak_loading_slots;
} shrike_streaming_statistics;
void shrike_slot_cache_statistics(shrike_slot_cache *cache, uint64_t expert_stride_bytes,
                                  shrike_streaming_statistics *out);
/* residentExperts, PreadExpertStreamer.swift:807-813: ascending ids; returns the count. */
size_t shrike_slot_cache_resident_experts(shrike_slot_cache *cache, int32_t *out, size_t capacity);
/* residencyEntry, PreadExpertStreamer.swift:663-670: state << 32 | cell. */
uint64_t shrike_slot_cache_entry(shrike_slot_cache *cache, uint32_t expert);
/* Entries whose word changed since the last drain, oldest first (an expert appears
 * once, with its latest word): what a caller mirrors into the device table with
 * shrike_hip_pool_table_publish. Returns the number written. */
size_t shrike_slot_cache_drain_publications(shrike_slot_cache *cache, uint32_t *experts,
                                            uint64_t *words, size_t capacity);

/* MoEExpertOffsets, sources/Shrike/Kernels/MoE/MoE.swift:4-39 (field for field). */
typedef struct {
    uint32_t gate_w_off, gate_s_off, gate_b_off;
    uint32_t up_w_off, up_s_off, up_b_off;
    uint32_t down_w_off, down_s_off, down_b_off;
    uint32_t gate_ab_off, up_ab_off, down_ab_off;
} shrike_expert_offsets;

/* ------------------------------------------------------- parallel expert reader */

/* The reference's reader interface, name for name
 * (sources/ShrikeKernelsC/include/shrike_expert_io.h:20-129; implementation
 * sources/ShrikeKernelsC/expert_io.c), for Linux: `threads` workers with a descriptor each
 * serve up to `batch_depth` published batches, oldest first; reads are plain pread, no
 * shared offset, no mmap. bypass_cache opens the descriptors with O_DIRECT (the reference
 * sets F_NOCACHE, expert_io.c:216-229) and, like the reference, fails the reader when the
 * file system refuses rather than read through the page cache; with it, destinations,
 * offsets and the stride must meet the device's direct-I/O alignment (the format's 16 KiB
 * does). create returns NULL and the cause in *out_errno; fetch returns 0 or the first
 * errno any worker saw (EIO for a blob that runs past the end of the file). */
typedef struct shrike_expert_reader shrike_expert_reader;
#define SHRIKE_IO_MAX_THREADS 16
#define SHRIKE_IO_MAX_BATCHES 2
shrike_expert_reader *shrike_expert_reader_create(const char *path, size_t expert_stride, int threads,
                                                  int batch_depth, int bypass_cache, int *out_errno);
/* no other thread may be inside a fetch when this runs (shrike_expert_io.h:58-60) */
void shrike_expert_reader_destroy(shrike_expert_reader *reader);
/* expert_ids[i] * expert_stride -> destinations[i], each expert_stride bytes; blocks until all landed */
int shrike_expert_reader_fetch(shrike_expert_reader *reader, const uint32_t *expert_ids,
                               void *const *destinations, size_t count);
/* the same with absolute byte offsets (shrike_expert_io.h:74-82) */
int shrike_expert_reader_fetch_offsets(shrike_expert_reader *reader, const uint64_t *offsets,
                                       void *const *destinations, size_t count);
int shrike_expert_reader_threads(const shrike_expert_reader *reader);
int shrike_expert_reader_batch_depth(const shrike_expert_reader *reader);

/* The claim, free-slot and cancel rules as pure functions (shrike_expert_io.h:90-129). */
typedef struct {
    int active;          /* published, not yet reaped by its submitter */
    uint64_t sequence;   /* publication order, lower is older */
    size_t next_index;   /* next unclaimed read */
    size_t count;        /* reads in the batch */
} shrike_expert_batch_slot;
int shrike_expert_reader_claim_slot(const shrike_expert_batch_slot *slots, int slot_count);
int shrike_expert_reader_free_slot(const shrike_expert_batch_slot *slots, int slot_count);
typedef struct {
    size_t count, next_index, outstanding;
    int first_errno;
} shrike_expert_batch_cancel_state;
void shrike_expert_reader_cancel_slot(shrike_expert_batch_cancel_state *slot);

/* ------------------------------------------------------- packed experts layout */

/* packed_experts/layout.json of a .gturbo model directory: the wire form
 * (sources/ShrikeFormat/GTurboPackedExpertsLayoutV1.swift:3-62), its structural validator
 * (:75-164), the manifest cross-check (:166-199) and the runtime view sorted by layer and by
 * logical expert id (sources/Shrike/Infrastructure/ModelIO/PackedExpertsLayout.swift:4-129).
 * decode: JSON text -> validated layout, NULL + EINVAL with the reference's field/reason in
 * shrike_host_last_error() otherwise. load: <model_dir>/packed_experts/layout.json; ENOENT
 * when missing, EFBIG when the file exceeds max_bytes ("exceeds metadata cap",
 * GTurboModelDirectory.swift:70-75; 0 = the format's 32 MiB). */
typedef struct shrike_packed_layout shrike_packed_layout;
#define SHRIKE_LAYOUT_ALIGNMENT_BYTES 16384u            /* GTurboFormatV1.alignmentBytes */
#define SHRIKE_LAYOUT_MAX_BYTES (32u * 1024u * 1024u)   /* GTurboFormatV1.residentIndexMaxBytes */
shrike_packed_layout *shrike_packed_layout_decode(const char *json, size_t bytes, int *out_errno);
shrike_packed_layout *shrike_packed_layout_load(const char *model_dir, uint64_t max_bytes, int *out_errno);
void shrike_packed_layout_destroy(shrike_packed_layout *layout);
const char *shrike_host_last_error(void);   /* of the calling thread; same text as shrike_hip_last_error */

uint64_t shrike_packed_layout_expert_stride(const shrike_packed_layout *layout);
int shrike_packed_layout_num_layers(const shrike_packed_layout *layout);
int shrike_packed_layout_experts_per_layer(const shrike_packed_layout *layout);
/* Layer `index` in ascending layer order: its id, file basename and expert count (0 for a
 * dense layer, which has no file). EINVAL past the end. */
int shrike_packed_layout_layer(const shrike_packed_layout *layout, int index, int *layer_id,
                               const char **file, int *expert_count);
/* PackedExpertsLayout.expert(layer:expert:) (PackedExpertsLayout.swift:53-65): position
 * `expert` in the layer's list sorted by logical id. ERANGE with the reference's wording
 * when either index is out of range. */
typedef struct {
    int32_t expert, physical_rank;
    uint64_t offset, size;      /* of the blob inside the layer file */
    uint32_t tensor_count;
} shrike_packed_expert;
int shrike_packed_layout_expert(const shrike_packed_layout *layout, int layer, int expert,
                                shrike_packed_expert *out);
/* A sub-tensor by role name ("gate", "gate_scales", ...). ENOENT when the blob has none. */
typedef struct {
    uint64_t offset, size;      /* relative to the blob */
    char dtype[8];              /* "U32" or "BF16" */
    uint32_t shape[4], rank;
    int32_t bits;               /* 0 when absent */
} shrike_packed_tensor;
int shrike_packed_layout_tensor(const shrike_packed_layout *layout, int layer, int expert,
                                const char *role, shrike_packed_tensor *out);
/* Model.routedExpertOffsets (sources/Shrike/Runtime/Inference/ModelExpertIO.swift:69-94): the
 * nine (+ three) offsets from expert 0 of the layer, 0 for a role the blob lacks; EINVAL
 * "is missing gate_bias" style when additive biases are expected and absent. */
int shrike_packed_layout_expert_offsets(const shrike_packed_layout *layout, int layer,
                                        int experts_have_additive_biases, shrike_expert_offsets *out);
/* crossValidate (GTurboPackedExpertsLayoutV1.swift:166-199) against a manifest's dimensions
 * and its file sizes ("packed_experts/<file>" paths). */
int shrike_packed_layout_cross_validate(const shrike_packed_layout *layout, int manifest_num_layers,
                                        int manifest_experts_per_layer, uint64_t manifest_expert_stride,
                                        const char *const *manifest_paths, const uint64_t *manifest_sizes,
                                        size_t manifest_file_count);

/* ------------------------------------------------------- routed tile loop of a streamed prefill chunk */

/* PrefillRoutedTileSchedulerConfig (sources/Shrike/Kernels/Prefill/MoE/PrefillRoutedTileScheduler.swift:46-96).
 * make clamps as the reference's init does: depth >= 1, 1...16 experts a tile, 1...16 tiles a
 * command buffer, lookahead 0 or 1 (reference defaults: 1, 8, 1, 0). */
typedef struct {
    int32_t max_pending_depth, tile_experts, tiles_per_command_buffer, fetch_lookahead;
} shrike_tile_scheduler_config;
void shrike_tile_scheduler_config_make(int max_pending_depth, int tile_experts, int tiles_per_command_buffer,
                                       int fetch_lookahead, shrike_tile_scheduler_config *out);
/* fitsSlotBudget (:63-66) and fitting (:71-91; 0 = nil, no configuration fits). */
int shrike_tile_scheduler_fits_slot_budget(const shrike_tile_scheduler_config *config, int slot_count, int reserved_hits);
int shrike_tile_scheduler_fitting(const shrike_tile_scheduler_config *config, int slot_count, int reserved_hits,
                                  shrike_tile_scheduler_config *out);
/* decide (:104-122). prefetchNext's avoidingSlots are the caller's pending slots, in their order.
 * pending_depth < 0: the input's default (1 with a pending tile, else 0). */
enum {
    SHRIKE_TILE_ISSUE_WITHOUT_PENDING = 0,
    SHRIKE_TILE_PREFETCH_NEXT = 1,
    SHRIKE_TILE_DRAIN_NO_ASSIGNED_SLOTS = 2,   /* drainBeforeIssue(.pendingTileHasNoAssignedSlots) */
    SHRIKE_TILE_DRAIN_PLAN_UNAVAILABLE = 3,    /* drainBeforeIssue(.avoidingSlotPlanUnavailable) */
    SHRIKE_TILE_DRAIN_MAX_DEPTH = 4            /* drainBeforeIssue(.maxPendingDepthReached) */
};
int shrike_tile_scheduler_decide(const shrike_tile_scheduler_config *config, int has_pending_tile, int pending_depth,
                                 size_t pending_assigned_slot_count, int avoiding_slot_plan_available);
int shrike_tile_scheduler_plans_lookahead(const shrike_tile_scheduler_config *config, int index, int tile_count);
int shrike_tile_scheduler_should_begin_lookahead(const shrike_tile_scheduler_config *config, int index, int tile_count,
                                                 int avoiding_slot_plan_available);
/* batchAction (:139-155) */
enum { SHRIKE_TILE_BATCH_OPEN = 0, SHRIKE_TILE_BATCH_FULL = 1, SHRIKE_TILE_BATCH_LAST_TILE = 2 };
typedef struct {
    int32_t commit_before_append;   /* the tile's plan collides with a slot the open batch still holds */
    int32_t commit_after_append;    /* SHRIKE_TILE_BATCH_* */
} shrike_tile_batch_action;
void shrike_tile_scheduler_batch_action(const shrike_tile_scheduler_config *config, int open_batch_tiles,
                                        size_t open_batch_slot_count, int next_tile_plan_available, int is_last_tile,
                                        shrike_tile_batch_action *out);

/* PrefillRoutedTileDriver (sources/Shrike/Kernels/Prefill/MoE/PrefillRoutedTileSequencer.swift:3-24) as
 * callbacks; those returning int give 0 or an error code, which ends the run. plan stores 0 in
 * *available when no plan avoiding the batches' slots (and those of the begun tile
 * avoiding_in_flight, -1 = none) fits the cache. */
typedef struct {
    void *context;
    int (*open_batch_tiles)(void *context);
    size_t (*open_batch_slot_count)(void *context);
    int (*pending_depth)(void *context);
    size_t (*pending_assigned_slot_count)(void *context);
    int (*plan)(void *context, int tile, int avoiding_in_flight, int *available);
    int (*begin)(void *context, int tile);
    int (*abandon_plan)(void *context, int tile);
    int (*encode)(void *context, int tile);
    void (*commit_open_batch)(void *context);
    int (*drain_oldest_batch)(void *context);
    void (*abandon_begun_fetches)(void *context);
} shrike_tile_driver;
/* PrefillRoutedTileSequencer.run (:30-85): a tile is awaited and encoded only once its successor's
 * fetch is in flight. On an error from a callback abandon_begun_fetches runs and the error returns. */
int shrike_tile_sequencer_run(const shrike_tile_scheduler_config *config, int tile_count, const shrike_tile_driver *driver);

/* PrefillChunkExpertProtection (sources/Shrike/Runtime/Inference/RealForwardRunner.swift:63-93): the chunk's
 * routed experts still to come are protected from eviction; planning a tile clears its own.
 * remaining: u8[experts_per_layer], 1 = protected. */
void shrike_chunk_protection_init(const int32_t *routed_experts, size_t count, uint8_t *remaining, size_t experts_per_layer);
void shrike_chunk_protection_planning(const int32_t *tile_experts, size_t count, uint8_t *remaining, size_t experts_per_layer);

/* PrefillStreamedTileSlotLifetime (sources/Shrike/Kernels/Prefill/MoE/PrefillGroupedRoutedMoE.swift:388-424):
 * a slot may not be planned again before the tile that holds it has completed. */
typedef struct shrike_tile_lifetime shrike_tile_lifetime;
enum {
    SHRIKE_TILE_LIFETIME_INVALID = -1,
    SHRIKE_TILE_LIFETIME_DUPLICATE_SLOTS = 1,
    SHRIKE_TILE_LIFETIME_SLOT_REUSE = 2,      /* slotReuseBeforeCompletion; *conflicting_tile names the holder */
    SHRIKE_TILE_LIFETIME_NOT_IN_FLIGHT = 3    /* completeWithoutInFlightTile */
};
shrike_tile_lifetime *shrike_tile_lifetime_create(void);
void shrike_tile_lifetime_destroy(shrike_tile_lifetime *lifetime);
int shrike_tile_lifetime_begin(shrike_tile_lifetime *lifetime, int tile_index, const int32_t *planned_slots, size_t count,
                               int *conflicting_tile);
int shrike_tile_lifetime_complete(shrike_tile_lifetime *lifetime, int tile_index);

/* ------------------------------------------------------- load operations and the predictive prefetch ring */

/* ExpertLoadOperation (sources/Shrike/Infrastructure/Streaming/ExpertLoadOperation.swift:3-153): one storage
 * batch whose submission is independent from its completion. Reference counted: create returns one
 * reference, the ring retains what is attached to its slots. finish(failure = 0) completes, any other
 * value fails the operation with that code; mark_in_flight and finish return EALREADY where the
 * reference traps a second start or a second completion. wait returns the failure code (0 = completed);
 * wait_until returns 1 once the operation is terminal, 0 at the deadline (shrike_monotonic_nanos clock). */
typedef struct shrike_load_operation shrike_load_operation;
enum { SHRIKE_LOAD_SUBMITTED = 0, SHRIKE_LOAD_IN_FLIGHT = 1, SHRIKE_LOAD_COMPLETED = 2, SHRIKE_LOAD_FAILED = 3 };
uint64_t shrike_monotonic_nanos(void);
shrike_load_operation *shrike_load_operation_create(void);
void shrike_load_operation_retain(shrike_load_operation *operation);
void shrike_load_operation_release(shrike_load_operation *operation);
int shrike_load_operation_state(shrike_load_operation *operation);
int shrike_load_operation_mark_in_flight(shrike_load_operation *operation);
int shrike_load_operation_finish(shrike_load_operation *operation, int failure);
int shrike_load_operation_wait(shrike_load_operation *operation);
int shrike_load_operation_wait_until(shrike_load_operation *operation, uint64_t deadline_nanos);
uint64_t shrike_load_operation_submitted_nanos(shrike_load_operation *operation);
uint64_t shrike_load_operation_started_nanos(shrike_load_operation *operation);
uint64_t shrike_load_operation_completed_nanos(shrike_load_operation *operation);

/* ExpertPrefetchStatistics (sources/Shrike/Runtime/Inference/ExpertPrefetchRing.swift:14-29), same fields. */
typedef struct {
    uint64_t issued, adopted, reclaimed, deferred, overlapped, late, joined, refused, failed, hook_failures,
        begin_nanos, leased_peak;
} shrike_prefetch_statistics;

/* ExpertPrefetchRing (ExpertPrefetchRing.swift:42-352). The ring owns `cells` of the expert pool (distinct,
 * at least one). drop(context, layer, expert, cell) removes a landing from its layer's residency table
 * and runs with the ring locked. issue(context, experts, cells, count, &operation) submits one read
 * of `count` experts into `cells` and returns 0 with the batch's operation (the ring retains it; the
 * caller keeps its own reference), SHRIKE_PREFETCH_CLAIM_REFUSED when the pool already holds one of the
 * experts (PrefetchClaimRefused: counted refused, begin returns 0), or an error code, which begin
 * returns after rolling the slots back. Results that the reference returns as dictionaries come back
 * as parallel arrays (room for as many entries as experts were passed), in slot order for ready_cells
 * and completion_nanos and in the experts' order for claim_demand. */
#define SHRIKE_PREFETCH_IN_FLIGHT_BUDGET 1            /* ExpertPrefetchRing.inFlightBudget (:49) */
#define SHRIKE_PREFETCH_ATTACH_SPIN_NANOS 5000000ull  /* ExpertPrefetchRing.attachSpinNanos (:48) */
#define SHRIKE_PREFETCH_CLAIM_REFUSED (-2)
typedef struct shrike_prefetch_ring shrike_prefetch_ring;
typedef void (*shrike_prefetch_drop)(void *context, int layer, int expert, int cell);
typedef int (*shrike_prefetch_issue)(void *context, const int *experts, const int *cells, size_t count,
                                     shrike_load_operation **out_operation);
shrike_prefetch_ring *shrike_prefetch_ring_create(const int *cells, size_t count, shrike_prefetch_drop drop, void *drop_context,
                                                  int *out_errno);                                            /* init (:95-102) */
void shrike_prefetch_ring_destroy(shrike_prefetch_ring *ring);
int shrike_prefetch_ring_begin(shrike_prefetch_ring *ring, int layer, const int *experts, size_t expert_count, const int *resident,
                               size_t resident_count, int deferred, shrike_prefetch_issue issue, void *issue_context); /* begin (:108-164) */
size_t shrike_prefetch_ring_ready_cells(shrike_prefetch_ring *ring, int layer, const int *experts, size_t expert_count,
                                        uint64_t join_nanos, int *out_experts, int *out_cells);               /* readyCells (:171-212) */
void shrike_prefetch_ring_consume(shrike_prefetch_ring *ring, int layer, const int *experts, size_t expert_count,
                                  const int *freed_experts, const int *freed_cells, size_t freed_count);      /* consume (:232-252) */
size_t shrike_prefetch_ring_claim_demand(shrike_prefetch_ring *ring, int layer, const int *experts, size_t expert_count,
                                         int *out_experts, int *out_cells);                                   /* claimDemand (:257-282) */
void shrike_prefetch_ring_attach_demand(shrike_prefetch_ring *ring, int layer, const int *experts, size_t expert_count,
                                        shrike_load_operation *operation);                                    /* attachDemand (:284-291) */
size_t shrike_prefetch_ring_completion_nanos(shrike_prefetch_ring *ring, int layer, const int *experts, size_t expert_count,
                                             int *out_experts, uint64_t *out_nanos);                          /* completionNanos (:293-304) */
void shrike_prefetch_ring_unlease(shrike_prefetch_ring *ring, int layer, const int *experts, size_t expert_count); /* :306-313 */
void shrike_prefetch_ring_note_demand_submission(shrike_prefetch_ring *ring);                                 /* :315-319 */
int shrike_prefetch_ring_note_hook_failure(shrike_prefetch_ring *ring);        /* 1 on the first failure (:322-327) */
void shrike_prefetch_ring_statistics(shrike_prefetch_ring *ring, shrike_prefetch_statistics *out);
int shrike_prefetch_ring_in_flight_count(shrike_prefetch_ring *ring);
int shrike_prefetch_ring_leased_count(shrike_prefetch_ring *ring);

/* ------------------------------------------------------- the CPU expert kernel */

/* shrike_int4_affine_gemv, sources/ShrikeKernelsC/include/shrike_kernels.h:9-29 (implementation
 * sources/ShrikeKernelsC/int4_affine_gemv.c:28-135), same name, arguments and meaning:
 * out[r] = sum_i (q[r][i] * scale[r][g(i)] + bias[r][g(i)]) * x[i] over a rows-by-n matrix of 4-bit codes, low nibble
 * first, one bf16 scale and one bf16 bias per group of 64; n a multiple of 64; out is written, not accumulated. The sum
 * is factored per group as scale * sum(q x) + bias * sum(x) and its additions run in the order of the reference's
 * portable branch (:114-134), whose bits the results are. Host memory only; thread-safe. */
void shrike_int4_affine_gemv(const uint8_t *weights, const uint16_t *scales, const uint16_t *biases, const float *x,
                             size_t rows, size_t n, float *out);
/* CPUExpertFFN.accumulate, sources/Shrike/Kernels/CPU/CPUExpertFFN.swift:102-140 (called at :82-90 by the CPU expert
 * workers): out[0..d) += route_weight * down(silu(gate . x) * (up . x)) for the expert blob at `expert` (bf16 metadata,
 * 4-bit codes), all in fp32. scratch: shrike_cpu_expert_ffn_scratch_floats(d, f) = 2 f + d floats, caller-owned. */
size_t shrike_cpu_expert_ffn_scratch_floats(uint32_t d, uint32_t f);
int shrike_cpu_expert_ffn_accumulate(const void *expert, const shrike_expert_offsets *offsets, const float *x, uint32_t d,
                                     uint32_t f, float route_weight, float *scratch, float *out);

/* ------------------------------------------------------- shared words between the host and the GPU */

/* sources/ShrikeKernelsC/include/shrike_atomics.h:7-14: an acquire load of a word a kernel writes while the host polls
 * it, a release store of a word the host publishes for a kernel to read. */
uint32_t shrike_load_acquire_u32(const uint32_t *word);
void shrike_store_release_u64(uint64_t *word, uint64_t value);

/* RouterHostReadback (sources/Shrike/Runtime/Inference/RouterHostReadback.swift:8-63): the host's half of the
 * classifier's tagged copy (the device's half is shrike_hip_moe_classify's host_readback operand). Every word carries
 * the launch's tag in its high 16 bits and a value in its low 16: the two counts, then five runs of top_k words (ids,
 * weight bits, hit positions, miss positions, predicted ids). The host polls the words while the command still runs
 * (RealForwardRunner.swift:3294) and trusts them only once every word carries the tag. */
typedef struct {
    uint32_t hit_count, miss_count;        /* clamped to top_k */
    uint32_t expert_ids[8];
    uint16_t weight_bits[8];
    uint32_t hit_positions[8];             /* the first hit_count are meaningful */
    uint32_t miss_positions[8];            /* the first miss_count are meaningful */
    uint32_t predicted_ids[8];
} shrike_router_readback;
uint32_t shrike_router_readback_word_count(uint32_t top_k);            /* wordCount(topK:), :24 */
uint32_t shrike_router_readback_word(uint32_t tag, uint32_t value);     /* word(tag:value:), :26-28 */
uint32_t shrike_router_readback_next_tag(uint32_t tag);                 /* nextTag(after:), :31-33: never 0, wraps at 16 bits */
int shrike_router_readback_is_complete(const uint32_t *words, uint32_t top_k, uint32_t tag);   /* isComplete, :35-41 */
/* decode, :43-62: 1 and *out filled when every word carries the tag, 0 (out untouched) otherwise. */
int shrike_router_readback_decode(const uint32_t *words, uint32_t top_k, uint32_t tag, shrike_router_readback *out);
/* The runner's wait (RealForwardRunner.swift:3294-3310): decode until it succeeds or shrike_monotonic_nanos() reaches
 * the deadline; 1 on success, 0 at the deadline. */
int shrike_router_readback_poll(const uint32_t *words, uint32_t top_k, uint32_t tag, uint64_t deadline_nanos,
                                shrike_router_readback *out);

/* ------------------------------------------------------- the storage submission service and its completion timeline */

/* ExpertIOScheduler (sources/Shrike/Infrastructure/Streaming/ExpertLoadOperation.swift:166-219): a fixed set of
 * submission threads over two queues; a queued demand batch runs before any queued speculative one. close runs what is
 * queued and ends the threads (submit then returns ESHUTDOWN); destroy closes first. work(context) runs on a worker. */
enum { SHRIKE_IO_DEMAND = 0, SHRIKE_IO_SPECULATIVE = 1 };  /* ExpertIOPriority, :166-169 */
typedef struct shrike_io_scheduler shrike_io_scheduler;
typedef void (*shrike_io_work)(void *context);
shrike_io_scheduler *shrike_io_scheduler_create(int worker_count, int *out_errno);   /* the reference's shared one has 4 */
int shrike_io_scheduler_submit(shrike_io_scheduler *scheduler, int priority, shrike_io_work work, void *context);
void shrike_io_scheduler_close(shrike_io_scheduler *scheduler);
void shrike_io_scheduler_destroy(shrike_io_scheduler *scheduler);
int shrike_io_scheduler_workers(const shrike_io_scheduler *scheduler);

/* ExpertIOEventCoordinator (sources/Shrike/Infrastructure/Streaming/ExpertIOEventCoordinator.swift:23-90): one timeline
 * for all expert reads of a model. reserve hands out the next value (never 0, never reused) and its status word, set to
 * 0 = loading; publish stores 1 = complete or 2 = failed and returns the timeline's published value, which moves only
 * over values whose predecessors are all terminal (an out-of-order completion is held). The status words are a ring of
 * word_count (0: SHRIKE_IO_STATUS_WORDS), a value's word at (value - 1) % word_count. status_words: caller-owned memory
 * the GPU can read (pinned host memory), or NULL for words of the timeline's own. A consumer on the GPU waits for value v
 * by waiting (hipStreamWaitEvent) for the event recorded behind v's copies and status store once published >= v says
 * that event and every earlier one is recorded, then reads the status word as the reference's kernels do. */
#define SHRIKE_IO_STATUS_WORDS 4096u  /* ExpertIOEventCoordinator.statusWordCount, :36 */
enum { SHRIKE_IO_STATUS_LOADING = 0, SHRIKE_IO_STATUS_COMPLETE = 1, SHRIKE_IO_STATUS_FAILED = 2 };
typedef struct shrike_io_timeline shrike_io_timeline;
typedef struct {
    uint64_t value;
    uint32_t status_index;     /* (value - 1) % word_count */
    uint32_t *status;          /* the word itself */
} shrike_io_completion_token;  /* ExpertIOCompletionToken, :7-15 */
shrike_io_timeline *shrike_io_timeline_create(uint32_t *status_words, uint32_t word_count, int *out_errno);
void shrike_io_timeline_destroy(shrike_io_timeline *timeline);
int shrike_io_timeline_reserve(shrike_io_timeline *timeline, shrike_io_completion_token *out);             /* reserve, :48-78 */
uint64_t shrike_io_timeline_publish(shrike_io_timeline *timeline, const shrike_io_completion_token *token, int succeeded); /* publish, :80-89 */
uint64_t shrike_io_timeline_published(shrike_io_timeline *timeline);  /* event.signaledValue */

#ifdef __cplusplus
}
#endif
#endif /* SHRIKE_HOST_H */
