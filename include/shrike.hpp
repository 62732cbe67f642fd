// C++ host side above the C ABI: the reference's operator classes with their method names and
// argument order (the reference's host is Swift; this is the same surface for a C++ host).
// Header only; every method forwards to one C entry point and throws shrike::Error with the
// library's message where the reference throws (runtime conditions) or traps (preconditions).
//
//   reference class                                   here
//   MoE (Kernels/MoE/MoE.swift)                       shrike::MoE
//   SharedExpertRuntime (Kernels/MoE/SharedExpert*)   shrike::MoE::encodeSharedExpert
//   ExpertCellArena + residency table                 shrike::ExpertPool
//   PreadExpertStreamer's cache planning              shrike::SlotCache
//   PrefillRouter / PrefillMoEGrouping /              shrike::PrefillRouter, shrike::PrefillMoEGrouping,
//   PrefillGroupedRoutedMoE / PrefillMoE              shrike::PrefillGroupedRoutedMoE, shrike::PrefillMoE
//   RuntimeConfiguration (budget -> slots)            shrike::RuntimeConfiguration
//   ParallelExpertReader (Infrastructure/Streaming)   shrike::ParallelExpertReader
//   PackedExpertsLayout(Reader) (Infrastructure/ModelIO) shrike::PackedExpertsLayout
//   PrefillRoutedTileScheduler / ...Sequencer / ...Driver shrike::PrefillRoutedTileScheduler, ...Sequencer, ...Driver
//   ExpertLoadOperation, ExpertPrefetchRing           shrike::ExpertLoadOperation, shrike::ExpertPrefetchRing
//   ExpertIOScheduler, ExpertIOEventCoordinator       shrike::ExpertIOScheduler, shrike::ExpertIOEventCoordinator
//   RouterHostReadback (Runtime/Inference)            shrike::RouterHostReadback
//   CPUExpertFFN (Kernels/CPU)                        shrike::CPUExpertFFN
#pragma once

#include <cerrno>
#include <condition_variable>
#include <cstdint>
#include <deque>
#include <exception>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <optional>
#include <stdexcept>
#include <string>
#include <thread>
#include <vector>

#include "shrike_hip.h"
#include "shrike_host.h"

namespace shrike {

struct Error : std::runtime_error {
    int code;
    Error(int c, const std::string &what) : std::runtime_error(what), code(c) {}
};
inline void check(int rc) {
    if (rc != 0) throw Error(rc, shrike_hip_last_error());
}

using Stream = void *;  // a hipStream_t; nullptr = the default stream

// RuntimeConfiguration.parseBudgetBytes / expertCacheSlots (RuntimeConfiguration.swift:111-149)
struct RuntimeConfiguration {
    static constexpr int64_t defaultExpertCacheBudgetBytes = int64_t(8) << 30;
    static std::optional<int64_t> parseBudgetBytes(const std::string &text) {
        const int64_t v = shrike_parse_budget_bytes(text.c_str());
        return v < 0 ? std::nullopt : std::optional<int64_t>(v);
    }
    static int expertCacheSlots(uint64_t expertStrideBytes, int layers, int64_t budgetBytes = defaultExpertCacheBudgetBytes) {
        return shrike_expert_cache_slots(expertStrideBytes, layers, budgetBytes);
    }
};

// MoEExpertOffsets / CPUExpertFFN.Offsets (MoE.swift:4-39, CPUExpertFFN.swift:34-61)
struct ExpertOffsets : shrike_expert_offsets {
    uint64_t strideBytes = 0;
    ExpertOffsets(uint32_t d, uint32_t f, uint32_t bits = 4, bool additiveBiases = false) {
        strideBytes = shrike_expert_offsets_make(d, f, bits, additiveBiases, this);
        if (!strideBytes) throw Error(EINVAL, "D and F must be positive multiples of 64, bits 4 or 8");
    }
};

// ExpertCellArena (ExpertCellArena.swift:16-133) with the streamer's residency table
class ExpertPool {
public:
    ExpertPool(uint32_t cellCount, uint64_t expertStride, uint32_t expertsPerLayer, uint64_t chunkBytes = 0) {
        int err = 0;
        h_ = shrike_hip_pool_create(cellCount, expertStride, expertsPerLayer, chunkBytes, &err);
        if (!h_) throw Error(err, shrike_hip_last_error());
    }
    // another layer's residency table over `arena`'s cells; `arena` must outlive it
    ExpertPool(const ExpertPool &arena, uint32_t expertsPerLayer) {
        int err = 0;
        h_ = shrike_hip_pool_create_layer_view(arena.h_, expertsPerLayer, &err);
        if (!h_) throw Error(err, shrike_hip_last_error());
    }
    ~ExpertPool() { shrike_hip_pool_destroy(h_); }
    ExpertPool(const ExpertPool &) = delete;
    ExpertPool &operator=(const ExpertPool &) = delete;
    uint64_t stride() const { return shrike_hip_pool_slot_stride(h_); }
    uint32_t cellCount() const { return shrike_hip_pool_cell_count(h_); }
    void *pointer(uint32_t cell) const { return shrike_hip_pool_cell_ptr(h_, cell); }
    const shrike_pool_bases *bases() const { return shrike_hip_pool_bases(h_); }
    const uint64_t *residencyTable() const { return static_cast<const uint64_t *>(shrike_hip_pool_residency_table(h_)); }
    void upload(uint32_t cell, const void *hostBlob, uint64_t bytes, Stream s) { check(shrike_hip_pool_upload_async(h_, cell, hostBlob, bytes, s)); }
    void publish(uint32_t expert, uint32_t cell, uint32_t state, Stream s) { check(shrike_hip_pool_table_publish(h_, expert, cell, state, s)); }
    // blobs at fileOffsets of the reader's layer file -> cells, through pinned staging memory
    void fetchExperts(shrike_expert_reader *reader, const std::vector<uint64_t> &fileOffsets, const std::vector<uint32_t> &cells,
                      uint64_t blobBytes, void *pinnedStaging, uint64_t stagingBytes, Stream s) {
        if (fileOffsets.size() != cells.size()) throw Error(EINVAL, "one cell per file offset");
        check(shrike_hip_pool_fetch_experts(h_, s, reader, fileOffsets.data(), cells.data(), uint32_t(cells.size()), blobBytes,
                                            pinnedStaging, stagingBytes));
    }
    uint64_t residencyEntry(uint32_t expert) const { return shrike_hip_pool_table_entry(h_, expert); }
    shrike_hip_pool *handle() const { return h_; }

private:
    shrike_hip_pool *h_;
};

// ParallelExpertReader (sources/Shrike/Infrastructure/Streaming/ParallelExpertReader.swift) over the
// reference's own C reader interface
class ParallelExpertReader {
public:
    struct Failure : Error {
        using Error::Error;
    };
    ParallelExpertReader(const std::string &path, size_t expertStride, int threads = 4, int batchDepth = 1, bool bypassCache = false) {
        int err = 0;
        h_ = shrike_expert_reader_create(path.c_str(), expertStride, threads, batchDepth, bypassCache, &err);
        if (!h_) throw Failure(err, "cannot open " + path);
    }
    ~ParallelExpertReader() { shrike_expert_reader_destroy(h_); }
    ParallelExpertReader(const ParallelExpertReader &) = delete;
    ParallelExpertReader &operator=(const ParallelExpertReader &) = delete;
    int threadCount() const { return shrike_expert_reader_threads(h_); }
    int batchDepth() const { return shrike_expert_reader_batch_depth(h_); }
    void fetch(const std::vector<uint32_t> &experts, const std::vector<void *> &into) {
        if (experts.size() != into.size()) throw Failure(EINVAL, "one destination per expert");
        if (int rc = shrike_expert_reader_fetch(h_, experts.data(), into.data(), experts.size())) throw Failure(rc, "expert read failed");
    }
    void fetch(const std::vector<uint64_t> &offsets, const std::vector<void *> &into) {
        if (offsets.size() != into.size()) throw Failure(EINVAL, "one destination per offset");
        if (int rc = shrike_expert_reader_fetch_offsets(h_, offsets.data(), into.data(), offsets.size())) throw Failure(rc, "expert read failed");
    }
    shrike_expert_reader *handle() const { return h_; }

private:
    shrike_expert_reader *h_;
};

// PackedExpertsLayout + PackedExpertsLayoutReader (PackedExpertsLayout.swift:34-129) and
// Model.routedExpertOffsets (ModelExpertIO.swift:69-94)
class PackedExpertsLayout {
public:
    static PackedExpertsLayout load(const std::string &modelDirectory, uint64_t maxBytes = 0) {
        int err = 0;
        shrike_packed_layout *h = shrike_packed_layout_load(modelDirectory.c_str(), maxBytes, &err);
        if (!h) throw Error(err, shrike_host_last_error());
        return PackedExpertsLayout(h);
    }
    static PackedExpertsLayout decode(const std::string &json) {
        int err = 0;
        shrike_packed_layout *h = shrike_packed_layout_decode(json.data(), json.size(), &err);
        if (!h) throw Error(err, shrike_host_last_error());
        return PackedExpertsLayout(h);
    }
    PackedExpertsLayout(PackedExpertsLayout &&o) noexcept : h_(o.h_) { o.h_ = nullptr; }
    PackedExpertsLayout(const PackedExpertsLayout &) = delete;
    PackedExpertsLayout &operator=(const PackedExpertsLayout &) = delete;
    ~PackedExpertsLayout() { shrike_packed_layout_destroy(h_); }
    uint64_t expertStride() const { return shrike_packed_layout_expert_stride(h_); }
    int numLayers() const { return shrike_packed_layout_num_layers(h_); }
    int expertsPerLayer() const { return shrike_packed_layout_experts_per_layer(h_); }
    std::string file(int layer) const {
        const char *name = nullptr;
        check(shrike_packed_layout_layer(h_, layer, nullptr, &name, nullptr));
        return name;
    }
    shrike_packed_expert expert(int layer, int expert) const {
        shrike_packed_expert out;
        check(shrike_packed_layout_expert(h_, layer, expert, &out));
        return out;
    }
    std::optional<shrike_packed_tensor> subTensor(int layer, int expert, const std::string &role) const {
        shrike_packed_tensor out;
        const int rc = shrike_packed_layout_tensor(h_, layer, expert, role.c_str(), &out);
        if (rc == ENOENT) return std::nullopt;
        check(rc);
        return out;
    }
    shrike_expert_offsets routedExpertOffsets(int layer, bool expertsHaveAdditiveBiases = false) const {
        shrike_expert_offsets out;
        check(shrike_packed_layout_expert_offsets(h_, layer, expertsHaveAdditiveBiases, &out));
        return out;
    }

private:
    explicit PackedExpertsLayout(shrike_packed_layout *h) : h_(h) {}
    shrike_packed_layout *h_;
};

struct PrefetchClaimRefused {  // PreadExpertStreamer.swift:46-49
    int expert, cell;
};

// ExpertCachePlan (PreadExpertStreamer.swift:17-38); assignedCells is the arena cell behind each
// assigned slot, what expertCachePlanBuffers binds
struct ExpertCachePlan {
    std::vector<int32_t> experts, assignedSlots;
    std::vector<uint64_t> assignedGenerations;
    std::vector<uint32_t> misses;
    uint32_t hits = 0;
    int32_t layer = 0;
    std::vector<uint32_t> assignedCells, adopted;
    std::map<int32_t, uint32_t> freedCells;
    shrike_expert_cache_plan raw() {
        return {uint32_t(experts.size()), layer, experts.data(), assignedSlots.data(), assignedGenerations.data(),
                misses.data(), uint32_t(misses.size()), hits, nullptr, nullptr, 0, 0, nullptr, nullptr};
    }
};

// ExpertCellArena's numbering and generations (ExpertCellArena.swift:16-29, :95-104)
class CellArena {
public:
    explicit CellArena(uint32_t cellCount) {
        int err = 0;
        h_ = shrike_cell_arena_create(cellCount, &err);
        if (!h_) throw Error(err, shrike_hip_last_error());
    }
    ~CellArena() { shrike_cell_arena_destroy(h_); }
    CellArena(const CellArena &) = delete;
    CellArena &operator=(const CellArena &) = delete;
    uint32_t cellCount() const { return shrike_cell_arena_cell_count(h_); }
    uint64_t cellGeneration(uint32_t cell) const { return shrike_cell_arena_generation(h_, cell); }
    shrike_cell_arena *handle() const { return h_; }

private:
    shrike_cell_arena *h_;
};

// The cache planning of PreadExpertStreamer (PreadExpertStreamer.swift:405-543, :676-767) with its
// landings and overflow slots (:815-1018)
class SlotCache {
public:
    SlotCache(uint32_t slotCount, uint32_t expertsPerLayer, uint32_t firstCell = 0, std::optional<double> slruProtectedShare = std::nullopt) {
        int err = 0;
        h_ = shrike_slot_cache_create(slotCount, expertsPerLayer, firstCell, slruProtectedShare ? SHRIKE_EVICT_SLRU : SHRIKE_EVICT_AGING_LFU,
                                      slruProtectedShare.value_or(0.0), &err);
        if (!h_) throw Error(err, shrike_hip_last_error());
    }
    // the slots take cells firstCell ..< firstCell + slotCount of a shared arena, which must outlive the cache
    SlotCache(CellArena &arena, uint32_t slotCount, uint32_t expertsPerLayer, uint32_t firstCell,
              std::optional<double> slruProtectedShare = std::nullopt) {
        int err = 0;
        h_ = shrike_slot_cache_create_in_arena(arena.handle(), slotCount, expertsPerLayer, firstCell,
                                               slruProtectedShare ? SHRIKE_EVICT_SLRU : SHRIKE_EVICT_AGING_LFU,
                                               slruProtectedShare.value_or(0.0), &err);
        if (!h_) throw Error(err, shrike_hip_last_error());
    }
    ~SlotCache() { shrike_slot_cache_destroy(h_); }
    SlotCache(const SlotCache &) = delete;
    SlotCache &operator=(const SlotCache &) = delete;

    // planExpertsCachedIfPossible: nullopt when the experts cannot be placed
    std::optional<ExpertCachePlan> planExpertsCachedIfPossible(const std::vector<int32_t> &experts, int32_t layer = 0,
                                                               const std::vector<int32_t> &avoidingSlots = {},
                                                               const std::vector<uint8_t> *protectedExperts = nullptr,
                                                               int64_t missesCounted = -1,
                                                               const std::vector<int32_t> &gpuMissedExperts = {},
                                                               const std::vector<int32_t> &leasedLandings = {}) {
        ExpertCachePlan p;
        const size_t n = experts.size();
        p.experts.resize(n);
        p.assignedSlots.resize(n);
        p.assignedGenerations.resize(n);
        p.misses.resize(n);
        p.assignedCells.resize(n);
        p.adopted.resize(n);
        std::vector<int32_t> freedExperts(n);
        std::vector<uint32_t> freedCells(n);
        shrike_expert_cache_plan raw = p.raw();
        raw.assigned_cells = p.assignedCells.data();
        raw.adopted = p.adopted.data();
        raw.freed_experts = freedExperts.data();
        raw.freed_cells = freedCells.data();
        const int rc = shrike_slot_cache_plan_with_landings(
            h_, experts.data(), uint32_t(n), layer, avoidingSlots.data(), uint32_t(avoidingSlots.size()),
            protectedExperts ? protectedExperts->data() : nullptr, protectedExperts ? uint32_t(protectedExperts->size()) : 0u,
            gpuMissedExperts.data(), uint32_t(gpuMissedExperts.size()), leasedLandings.data(), uint32_t(leasedLandings.size()),
            missesCounted, &raw);
        if (rc == ENOSPC) return std::nullopt;
        check(rc);
        p.misses.resize(raw.miss_count);
        p.adopted.resize(raw.adopted_count);
        for (uint32_t i = 0; i < raw.freed_count; ++i) p.freedCells[freedExperts[i]] = freedCells[i];
        p.hits = raw.hits;
        p.layer = raw.layer;
        return p;
    }
    // planExpertsCached: throws ModelError.expertCacheUnplaceable's counterpart
    ExpertCachePlan planExpertsCached(const std::vector<int32_t> &experts, int32_t layer = 0, const std::vector<int32_t> &avoidingSlots = {},
                                      const std::vector<uint8_t> *protectedExperts = nullptr) {
        auto p = planExpertsCachedIfPossible(experts, layer, avoidingSlots, protectedExperts);
        if (!p) throw Error(ENOSPC, shrike_hip_last_error());
        return *p;
    }
    void markPlanMissesResident(ExpertCachePlan &plan, uint64_t elapsedNanos = 0, uint64_t fetchNanos = 0) {
        shrike_expert_cache_plan raw = plan.raw();
        check(shrike_slot_cache_complete(h_, &raw, elapsedNanos, fetchNanos));
    }
    void abandonExpertCachePlan(ExpertCachePlan &plan) {
        shrike_expert_cache_plan raw = plan.raw();
        shrike_slot_cache_abandon(h_, &raw);
    }
    void pin(ExpertCachePlan &plan) {
        shrike_expert_cache_plan raw = plan.raw();
        check(shrike_slot_cache_pin(h_, &raw));
    }
    void unpin(const ExpertCachePlan &plan) {
        shrike_slot_cache_unpin(h_, plan.assignedSlots.data(), plan.assignedGenerations.data(), uint32_t(plan.assignedSlots.size()));
    }
    shrike_streaming_statistics statistics(uint64_t expertStrideBytes = 0) {
        shrike_streaming_statistics s{};
        shrike_slot_cache_statistics(h_, expertStrideBytes, &s);
        return s;
    }
    std::vector<int32_t> residentExperts(size_t capacity = 4096) {
        std::vector<int32_t> out(capacity);
        out.resize(shrike_slot_cache_resident_experts(h_, out.data(), capacity));
        return out;
    }
    uint64_t residencyEntry(uint32_t expert) { return shrike_slot_cache_entry(h_, expert); }

    // landings, PreadExpertStreamer.swift:815-852, :1010-1018
    bool claimLanding(int32_t expert, int64_t cell) { return shrike_slot_cache_claim_landing(h_, expert, cell) != 0; }
    bool completeLanding(int32_t expert, int64_t cell) { return shrike_slot_cache_complete_landing(h_, expert, cell) != 0; }
    void failLanding(int32_t expert, int64_t cell) { shrike_slot_cache_fail_landing(h_, expert, cell); }
    void dropLanding(int32_t expert, int64_t cell) { shrike_slot_cache_drop_landing(h_, expert, cell); }
    // the claims of beginPrefetch (:1034-1057); throws PrefetchClaimRefused when the pool holds a predicted expert
    void claimPrefetch(const std::vector<int32_t> &experts, const std::vector<int64_t> &cells) {
        if (experts.size() != cells.size()) throw Error(EINVAL, "prefetch experts and cells differ in count");
        uint32_t refused = 0;
        const int rc = shrike_slot_cache_claim_prefetch(h_, experts.data(), cells.data(), uint32_t(experts.size()), &refused);
        if (rc == SHRIKE_PREFETCH_CLAIM_REFUSED) throw PrefetchClaimRefused{int(experts[refused]), int(cells[refused])};
        check(rc);
    }
    // overflow slots, :860-893, :968-993; reserveOverflowSlot gives the cell
    std::optional<uint32_t> reserveOverflowSlot(int32_t expert, const std::vector<int32_t> &protecting = {}) {
        const int64_t cell = shrike_slot_cache_reserve_overflow_slot(h_, expert, protecting.data(), uint32_t(protecting.size()));
        if (cell < 0) return std::nullopt;
        return uint32_t(cell);
    }
    void abandonOverflowSlot(int32_t expert, int64_t cell) { shrike_slot_cache_abandon_overflow_slot(h_, expert, cell); }
    // the completion of beginAgreedReads, :936-964
    void finishAgreedReads(const std::vector<int32_t> &experts, const std::vector<int64_t> &cells, bool succeeded,
                           uint64_t elapsedNanos = 0, uint64_t fetchNanos = 0) {
        if (experts.size() != cells.size()) throw Error(EINVAL, "agreed reads' experts and cells differ in count");
        check(shrike_slot_cache_finish_agreed_reads(h_, experts.data(), cells.data(), uint32_t(experts.size()), succeeded,
                                                    elapsedNanos, fetchNanos));
    }
    int64_t slotCell(uint32_t slot) { return shrike_slot_cache_slot_cell(h_, slot); }
    bool ownsCell(uint32_t cell) { return shrike_slot_cache_owns_cell(h_, cell) != 0; }
    // mirrors every changed residency word into the pool's device table, in order, on `s`
    void publishTo(ExpertPool &pool, Stream s, size_t expertsPerLayer) {
        std::vector<uint32_t> ids(expertsPerLayer);
        std::vector<uint64_t> words(expertsPerLayer);
        const size_t n = shrike_slot_cache_drain_publications(h_, ids.data(), words.data(), ids.size());
        for (size_t i = 0; i < n; ++i) pool.publish(ids[i], uint32_t(words[i]), uint32_t(words[i] >> 32), s);
    }

private:
    shrike_slot_cache *h_;
};

// MoE (MoE.swift:41-216): enqueue-only operators on a stream
class MoE {
public:
    explicit MoE(const shrike_moe_desc &desc) {
        int err = 0;
        h_ = shrike_hip_moe_create(&desc, &err);
        if (!h_) throw Error(err, shrike_hip_last_error());
    }
    ~MoE() { shrike_hip_moe_destroy(h_); }
    MoE(const MoE &) = delete;
    MoE &operator=(const MoE &) = delete;
    shrike_hip_moe *handle() const { return h_; }

    void encodeRouter(Stream s, const void *weights, const void *scales, const void *biases, const void *hidden,
                      const void *effectiveScale, const void *perExpertScale, const void *logitBias, uint32_t *outIndices,
                      void *outWeights, uint32_t numExperts, uint32_t d, uint32_t topK) {  // MoE.swift:249-261
        check(shrike_hip_moe_router(h_, s, weights, scales, biases, hidden, effectiveScale, perExpertScale, logitBias, outIndices,
                                    outWeights, numExperts, d, topK));
    }
    void encodeResidencyClassification(Stream s, const uint32_t *topKIndices, const uint64_t *residency, uint32_t *hitCount,
                                       uint32_t *hitPositions, uint32_t *missCount, uint32_t *missPositions, uint32_t *missExperts,
                                       uint32_t *resolvedSlots, uint32_t topK, uint32_t numExperts, const uint32_t fullGrids[12],
                                       uint32_t *specArgs, uint32_t *hostReadback = nullptr, uint32_t readbackTag = 0,
                                       const void *topKWeights = nullptr, const uint32_t *predicted = nullptr) {  // MoE.swift:552-566
        check(shrike_hip_moe_classify(h_, s, topKIndices, residency, hitCount, hitPositions, missCount, missPositions, missExperts,
                                      resolvedSlots, topK, numExperts, fullGrids, specArgs, hostReadback, readbackTag, topKWeights,
                                      predicted));
    }
    void encodeSpecPhase1U16Load(Stream s, const ExpertPool &pool, const uint32_t *resolvedSlots, const shrike_expert_offsets &offsets,
                                 const void *x, void *acts, uint32_t d, uint32_t f, uint32_t topK, const uint32_t *indirect = nullptr,
                                 const uint32_t *ioStatus = nullptr) {  // MoE.swift:906-923
        check(shrike_hip_moe_phase1_pool(h_, s, pool.bases(), pool.stride(), resolvedSlots, &offsets, x, acts, d, f, topK, indirect, ioStatus));
    }
    void encodeSpecPhase2Reduce(Stream s, const ExpertPool &pool, const uint32_t *resolvedSlots, const uint32_t *fallbackCells,
                                const shrike_expert_offsets &offsets, const void *acts, const void *routingWeights, const void *residual,
                                void *y, void *hidden, uint32_t d, uint32_t f, uint32_t topK, const uint32_t *indirect = nullptr,
                                const uint32_t *ioStatus = nullptr) {  // MoE.swift:992-1014
        check(shrike_hip_moe_phase2_pool(h_, s, pool.bases(), pool.stride(), resolvedSlots, fallbackCells, &offsets, acts, routingWeights,
                                         residual, y, hidden, d, f, topK, indirect, ioStatus));
    }
    // MoE.swift:651-665 and, with activeSlots, :694-712: the route's blobs named by a device array of pointers
    void encodeRoutedPersistentPhase1U16Load(Stream s, const void *const *routedArgBuffer, const shrike_expert_offsets &offsets,
                                             const void *x, void *acts, uint32_t d, uint32_t f, uint32_t topK,
                                             const uint32_t *ioStatus = nullptr) {
        check(shrike_hip_moe_phase1_blobs(h_, s, routedArgBuffer, &offsets, x, acts, d, f, topK, nullptr, 0, ioStatus));
    }
    void encodeRoutedPersistentPhase1SubsetU16Load(Stream s, const void *const *routedArgBuffer, const shrike_expert_offsets &offsets,
                                                   const void *x, void *acts, const uint32_t *activeSlots, uint32_t activeCount,
                                                   uint32_t d, uint32_t f, uint32_t topK, const uint32_t *ioStatus = nullptr) {
        if (activeCount == 0) return;  // MoE.swift:710
        check(shrike_hip_moe_phase1_blobs(h_, s, routedArgBuffer, &offsets, x, acts, d, f, topK, activeSlots, activeCount, ioStatus));
    }
    void encodeRoutedPersistentPhase2Reduce(Stream s, const void *const *routedArgBuffer, const shrike_expert_offsets &offsets,
                                            const void *acts, const void *routingWeights, const void *residual, void *y, void *hidden,
                                            uint32_t d, uint32_t f, uint32_t topK, const uint32_t *ioStatus = nullptr) {  // MoE.swift:816-836
        check(shrike_hip_moe_phase2_blobs(h_, s, routedArgBuffer, &offsets, acts, routingWeights, residual, y, hidden, d, f, topK, ioStatus));
    }
    void encodeSharedExpert(Stream s, const shrike_projection &gate, const shrike_projection &up, const shrike_projection &down,
                            uint32_t bits, const void *x, void *scratch, void *h1, const void *scalarGate, uint32_t d, uint32_t fShared) {
        check(shrike_hip_shared_expert(h_, s, &gate, &up, &down, bits, x, scratch, h1, scalarGate, d, fShared));
    }
    void encodeDecodeLayer(Stream s, const shrike_decode_layer_args &args) { check(shrike_hip_moe_decode_layer(h_, s, &args)); }
    // the same for several sequences, one token each (rows of x xStrideElements apart)
    void encodeDecodeLayerBatch(Stream s, const shrike_decode_layer_args &args, uint32_t tokens, uint32_t xStrideElements) {
        check(shrike_hip_moe_decode_layer_batch(h_, s, &args, tokens, xStrideElements));
    }

private:
    shrike_hip_moe *h_;
};

// PrefillRouter (PrefillRouter.swift:41-152)
struct PrefillRouter {
    static constexpr int tokenBlock = 12;
    static size_t workspaceBytes(uint32_t queryCount, uint32_t numExperts, uint32_t d) {
        return shrike_hip_prefill_router_workspace_bytes(queryCount, numExperts, d);
    }
    static void encodeBlock(MoE &moe, Stream s, const void *weights, const void *scales, const void *biases, const void *hidden,
                            const void *effectiveScale, const void *perExpertScale, const void *logitBias, uint32_t *outIndices,
                            void *outWeights, float *workspace, uint32_t queryCount, uint32_t numExperts, uint32_t d, uint32_t topK,
                            uint32_t hiddenStrideElements) {
        check(shrike_hip_prefill_router(moe.handle(), s, weights, scales, biases, hidden, effectiveScale, perExpertScale, logitBias,
                                        outIndices, outWeights, workspace, queryCount, numExperts, d, topK, hiddenStrideElements));
    }
    // the same, leaving the group sums of `hidden` at the head of the grouped FFN's workspace (no counterpart in the
    // reference: a runner that hands both operators the same rows reads them once)
    static void encodeBlockWithGroupSums(MoE &moe, Stream s, const void *weights, const void *scales, const void *biases, const void *hidden,
                                         const void *effectiveScale, const void *perExpertScale, const void *logitBias, uint32_t *outIndices,
                                         void *outWeights, float *workspace, uint32_t queryCount, uint32_t numExperts, uint32_t d,
                                         uint32_t topK, uint32_t hiddenStrideElements, void *ffnWorkspace) {
        check(shrike_hip_prefill_router_with_group_sums(moe.handle(), s, weights, scales, biases, hidden, effectiveScale, perExpertScale,
                                                        logitBias, outIndices, outWeights, workspace, queryCount, numExperts, d, topK,
                                                        hiddenStrideElements, ffnWorkspace));
    }
    static std::vector<shrike_token_expert_pair> makeTokenExpertPairs(const std::vector<uint32_t> &indices, const std::vector<uint16_t> &weights,
                                                                      uint32_t queryCount, uint32_t topK) {
        if (indices.size() != size_t(queryCount) * topK || weights.size() != indices.size()) throw Error(EINVAL, "indices count mismatch");
        std::vector<shrike_token_expert_pair> pairs(indices.size());
        check(shrike_make_token_expert_pairs(indices.data(), weights.data(), queryCount, topK, pairs.data()));
        return pairs;
    }
};

// PrefillMoEGroupedRoutes and PrefillMoEGrouping.groupTokenExpertPairs (PrefillMoEGrouping.swift:32-50, :269-370)
struct PrefillMoEGroupedRoutes {
    std::vector<shrike_token_expert_pair> sortedPairs;
    std::vector<uint32_t> perExpertOffsets, perExpertCounts;
    std::vector<shrike_moe_group> groups;
    std::vector<shrike_moe_tile> tiles;
    int64_t queryCount = 0;
    uint32_t maxPairsPerExpert = 0, maxPairsPerTile = 0, maxLiveExpertsPerTile = 0;
};
struct GroupingError : Error {
    int64_t values[2];
    GroupingError(int code, const int64_t v[2]) : Error(code, shrike_hip_last_error()) { values[0] = v[0]; values[1] = v[1]; }
};
struct PrefillMoEGrouping {
    static PrefillMoEGroupedRoutes groupTokenExpertPairs(const std::vector<shrike_token_expert_pair> &pairs, int64_t queryCount, int64_t topK,
                                                         int64_t numExperts, int64_t tileExpertCount = 16,
                                                         const std::vector<uint64_t> *expertSortKeys = nullptr) {
        PrefillMoEGroupedRoutes r;
        const size_t e = numExperts > 0 ? size_t(numExperts) : 1, cap = std::max<size_t>(1, std::min(e, pairs.size()));
        r.sortedPairs.resize(std::max<size_t>(1, pairs.size()));
        r.perExpertOffsets.resize(e);
        r.perExpertCounts.resize(e);
        r.groups.resize(cap);
        r.tiles.resize(cap);
        shrike_grouped_routes out{r.sortedPairs.data(), r.perExpertOffsets.data(), r.perExpertCounts.data(), r.groups.data(), r.tiles.data()};
        const int rc = shrike_group_pairs(pairs.data(), pairs.size(), queryCount, topK, numExperts, tileExpertCount,
                                          expertSortKeys ? expertSortKeys->data() : nullptr, expertSortKeys ? expertSortKeys->size() : 0, &out);
        if (rc != 0) throw GroupingError(rc, out.error_value);
        r.sortedPairs.resize(pairs.size());
        r.perExpertOffsets.resize(size_t(numExperts));
        r.perExpertCounts.resize(size_t(numExperts));
        r.groups.resize(out.group_count);
        r.tiles.resize(out.tile_count);
        r.queryCount = queryCount;
        r.maxPairsPerExpert = out.max_pairs_per_expert;
        r.maxPairsPerTile = out.max_pairs_per_tile;
        r.maxLiveExpertsPerTile = out.max_live_experts_per_tile;
        return r;
    }
    // the same permutation on the device, from the router's token-major output
    static void encodeGroupPairs(Stream s, const uint32_t *indices, const void *weights, uint32_t queryCount, uint32_t topK, uint32_t numExperts,
                                 const uint64_t *expertSortKeys, const uint64_t *residency, const shrike_hip_grouped_routes &out) {
        check(shrike_hip_group_pairs(s, indices, weights, queryCount, topK, numExperts, expertSortKeys, residency, &out));
    }
};

// PrefillSweepOrder (PrefillMoEGrouping.swift:91-266)
struct PrefillSweepOrder {
    static std::vector<uint32_t> residentFirstBalanced(const std::vector<uint32_t> &experts, const std::vector<int64_t> &rows,
                                                       const std::vector<int64_t> &lastRow, const std::vector<uint8_t> &resident, int64_t slots,
                                                       int64_t tileWidth) {
        std::vector<uint32_t> order(std::max<size_t>(1, experts.size()));
        size_t n = 0;
        check(shrike_sweep_order_resident_first_balanced(experts.data(), rows.data(), lastRow.data(), experts.size(), resident.data(),
                                                         resident.size(), slots, tileWidth, order.data(), &n));
        order.resize(n);
        return order;
    }
    static std::vector<uint64_t> expertSortKeys(const std::vector<uint32_t> &order, size_t numExperts) {
        std::vector<uint64_t> keys(std::max<size_t>(1, numExperts));
        shrike_expert_sort_keys(order.data(), order.size(), numExperts, keys.data());
        keys.resize(numExperts);
        return keys;
    }
};

// PrefillGroupedRoutedMoE (PrefillGroupedRoutedMoE.swift:104-284, :925-939)
struct PrefillRoutedExpertWave {
    std::vector<shrike_routed_expert_block> blocks;
    int paddedRows = 0, tailRows = 0;
};
struct PrefillGroupedRoutedMoE {
    static constexpr int groupedRowTile = 64, groupedTailRowTile = 32;
    static std::vector<PrefillRoutedExpertWave> planExpertWaves(const std::vector<shrike_expert_pair_range> &ranges,
                                                                const std::vector<uint32_t> &boundExperts, int64_t stagingRows,
                                                                int64_t rowTile = groupedRowTile, int64_t tailTile = 0) {
        std::vector<shrike_routed_expert_block> blocks(64);
        std::vector<shrike_routed_expert_wave> waves(16);
        size_t nb = 0, nw = 0;
        for (;;) {
            const int rc = shrike_plan_expert_waves(ranges.data(), ranges.size(), boundExperts.data(), boundExperts.size(), stagingRows, rowTile,
                                                    tailTile, blocks.data(), blocks.size(), &nb, waves.data(), waves.size(), &nw);
            if (rc == ENOSPC) {
                blocks.resize(std::max(blocks.size(), nb));
                waves.resize(std::max(waves.size(), nw));
                continue;
            }
            check(rc);
            break;
        }
        std::vector<PrefillRoutedExpertWave> out(nw);
        for (size_t i = 0; i < nw; ++i) {
            out[i].blocks.assign(blocks.begin() + waves[i].block_start, blocks.begin() + waves[i].block_start + waves[i].block_count);
            out[i].paddedRows = int(waves[i].padded_rows);
            out[i].tailRows = int(waves[i].tail_rows);
        }
        return out;
    }
    static std::vector<uint32_t> rowTileTable(const PrefillRoutedExpertWave &wave, uint32_t rowTile = groupedRowTile) {
        std::vector<uint32_t> table(std::max<size_t>(1, size_t(wave.paddedRows) / rowTile));
        check(shrike_row_tile_table(wave.blocks.data(), wave.blocks.size(), uint32_t(wave.paddedRows), rowTile, table.data()));
        table.resize(size_t(wave.paddedRows) / rowTile);
        return table;
    }
    static size_t workspaceBytes(uint32_t queryCount, uint32_t maxRowTiles, uint32_t d, uint32_t f) {
        return shrike_hip_prefill_ffn_workspace_bytes(queryCount, maxRowTiles, d, f);
    }
    static void encodeGroupedExpertGEMMs(MoE &moe, Stream s, const ExpertPool &pool, const shrike_expert_offsets &offsets,
                                         const shrike_hip_grouped_routes &routes, uint32_t maxRowTiles, const void *hidden,
                                         uint32_t hiddenStrideElements, void *routePartials, void *workspace, size_t workspaceSize,
                                         uint32_t queryCount, uint32_t d, uint32_t f, uint32_t topK) {
        check(shrike_hip_prefill_grouped_ffn(moe.handle(), s, pool.bases(), pool.stride(), &offsets, &routes, maxRowTiles, hidden,
                                             hiddenStrideElements, routePartials, workspace, workspaceSize, queryCount, d, f, topK));
    }
    // the same for a workspace whose head holds the group sums PrefillRouter::encodeBlockWithGroupSums left there
    static void encodeGroupedExpertGEMMsPresummed(MoE &moe, Stream s, const ExpertPool &pool, const shrike_expert_offsets &offsets,
                                                  const shrike_hip_grouped_routes &routes, uint32_t maxRowTiles, const void *hidden,
                                                  uint32_t hiddenStrideElements, void *routePartials, void *workspace, size_t workspaceSize,
                                                  uint32_t queryCount, uint32_t d, uint32_t f, uint32_t topK) {
        check(shrike_hip_prefill_grouped_ffn_presummed(moe.handle(), s, pool.bases(), pool.stride(), &offsets, &routes, maxRowTiles,
                                                       hidden, hiddenStrideElements, routePartials, workspace, workspaceSize, queryCount,
                                                       d, f, topK));
    }
    // encodeStreamedBatched (PrefillGroupedRoutedMoE.swift:846-922): the sorted pairs [pairStart, pairStart + pairCount)
    // against `residency` (device table, or null for the cells recorded at grouping); returns the microbatch count
    static uint32_t encodeStreamedBatched(MoE &moe, Stream s, const ExpertPool &pool, const shrike_expert_offsets &offsets,
                                          const shrike_hip_grouped_routes &routes, uint32_t maxRowTiles, const uint64_t *residency,
                                          uint32_t pairStart, uint32_t pairCount, const void *hidden, uint32_t hiddenStrideElements,
                                          void *routePartials, void *workspace, size_t workspaceSize, uint32_t queryCount,
                                          uint32_t d, uint32_t f, uint32_t topK, uint32_t pairMicrobatchRows = 32) {
        uint32_t microbatches = 0;
        check(shrike_hip_prefill_streamed_batched(moe.handle(), s, pool.bases(), pool.stride(), &offsets, &routes, maxRowTiles,
                                                  residency, pairStart, pairCount, pairMicrobatchRows, hidden, hiddenStrideElements,
                                                  routePartials, workspace, workspaceSize, queryCount, d, f, topK, &microbatches));
        return microbatches;
    }
};

// PrefillMoE (PrefillMoE.swift:11-40)
struct PrefillMoE {
    static void encodeReduceTokenMajor(Stream s, const void *routePartials, const void *routeWeights, void *h2, uint32_t queryCount,
                                       uint32_t topK, uint32_t d) {
        check(shrike_hip_prefill_reduce(s, routePartials, routeWeights, h2, queryCount, topK, d));
    }
    static void encodeResidualAdd(Stream s, void *hidden, const void *delta, uint64_t count) {
        check(shrike_hip_residual_add_f16(s, hidden, delta, count));
    }
};

// PrefillRoutedTileSchedulerConfig / PrefillRoutedTileScheduler (PrefillRoutedTileScheduler.swift:46-155)
struct PrefillRoutedTileSchedulerConfig : shrike_tile_scheduler_config {
    explicit PrefillRoutedTileSchedulerConfig(int maxPendingDepth = 1, int tileExperts = 8, int tilesPerCommandBuffer = 1,
                                              int fetchLookahead = 0) {
        shrike_tile_scheduler_config_make(maxPendingDepth, tileExperts, tilesPerCommandBuffer, fetchLookahead, this);
    }
    bool fitsSlotBudget(int slotCount, int reservedHits = 0) const {
        return shrike_tile_scheduler_fits_slot_budget(this, slotCount, reservedHits) != 0;
    }
    std::optional<PrefillRoutedTileSchedulerConfig> fitting(int slotCount, int reservedHits = 0) const {
        PrefillRoutedTileSchedulerConfig out;
        if (!shrike_tile_scheduler_fitting(this, slotCount, reservedHits, &out)) return std::nullopt;
        return out;
    }
};

struct PrefillRoutedTileScheduler {
    PrefillRoutedTileSchedulerConfig config;
    // SHRIKE_TILE_ISSUE_WITHOUT_PENDING ... SHRIKE_TILE_DRAIN_MAX_DEPTH; pendingDepth < 0 = the input's default
    int decide(bool hasPendingTile, size_t pendingAssignedSlotCount, bool avoidingSlotPlanAvailable, int pendingDepth = -1) const {
        return shrike_tile_scheduler_decide(&config, hasPendingTile, pendingDepth, pendingAssignedSlotCount, avoidingSlotPlanAvailable);
    }
    shrike_tile_batch_action batchAction(int openBatchTiles, size_t openBatchSlotCount, bool nextTilePlanAvailable, bool isLastTile) const {
        shrike_tile_batch_action out;
        shrike_tile_scheduler_batch_action(&config, openBatchTiles, openBatchSlotCount, nextTilePlanAvailable, isLastTile, &out);
        return out;
    }
    bool shouldBeginLookahead(int index, int tileCount, bool avoidingSlotPlanAvailable) const {
        return shrike_tile_scheduler_should_begin_lookahead(&config, index, tileCount, avoidingSlotPlanAvailable) != 0;
    }
};

// PrefillRoutedTileDriver (PrefillRoutedTileSequencer.swift:3-24): what the sequencer drives. Methods may throw.
struct PrefillRoutedTileDriver {
    virtual ~PrefillRoutedTileDriver() = default;
    virtual int openBatchTiles() = 0;
    virtual size_t openBatchSlotCount() = 0;
    virtual int pendingDepth() = 0;
    virtual size_t pendingAssignedSlotCount() = 0;
    virtual bool plan(int tile, std::optional<int> avoidingInFlight) = 0;
    virtual void begin(int tile) = 0;
    virtual void abandonPlan(int tile) = 0;
    virtual void encode(int tile) = 0;
    virtual void commitOpenBatch() = 0;
    virtual void drainOldestBatch() = 0;
    virtual void abandonBegunFetches() = 0;
};

// PrefillRoutedTileSequencer (PrefillRoutedTileSequencer.swift:26-104); a driver's exception crosses the C
// boundary as a code and is rethrown here, after abandonBegunFetches has run.
struct PrefillRoutedTileSequencer {
    PrefillRoutedTileScheduler scheduler;
    void run(int tileCount, PrefillRoutedTileDriver &driver) const {
        Box box{&driver, nullptr};
        shrike_tile_driver d = {};
        d.context = &box;
        d.open_batch_tiles = [](void *c) { return static_cast<Box *>(c)->driver->openBatchTiles(); };
        d.open_batch_slot_count = [](void *c) { return static_cast<Box *>(c)->driver->openBatchSlotCount(); };
        d.pending_depth = [](void *c) { return static_cast<Box *>(c)->driver->pendingDepth(); };
        d.pending_assigned_slot_count = [](void *c) { return static_cast<Box *>(c)->driver->pendingAssignedSlotCount(); };
        d.plan = [](void *c, int tile, int avoiding, int *available) {
            return call(c, [&](PrefillRoutedTileDriver &drv) {
                *available = drv.plan(tile, avoiding < 0 ? std::nullopt : std::optional<int>(avoiding)) ? 1 : 0;
            });
        };
        d.begin = [](void *c, int tile) { return call(c, [&](PrefillRoutedTileDriver &drv) { drv.begin(tile); }); };
        d.abandon_plan = [](void *c, int tile) { return call(c, [&](PrefillRoutedTileDriver &drv) { drv.abandonPlan(tile); }); };
        d.encode = [](void *c, int tile) { return call(c, [&](PrefillRoutedTileDriver &drv) { drv.encode(tile); }); };
        d.commit_open_batch = [](void *c) { static_cast<Box *>(c)->driver->commitOpenBatch(); };
        d.drain_oldest_batch = [](void *c) { return call(c, [&](PrefillRoutedTileDriver &drv) { drv.drainOldestBatch(); }); };
        d.abandon_begun_fetches = [](void *c) { static_cast<Box *>(c)->driver->abandonBegunFetches(); };
        const int rc = shrike_tile_sequencer_run(&scheduler.config, tileCount, &d);
        if (box.failure) std::rethrow_exception(box.failure);
        check(rc);
    }

private:
    struct Box {
        PrefillRoutedTileDriver *driver;
        std::exception_ptr failure;
    };
    template <class Body>
    static int call(void *ctx, Body &&body) {
        Box *b = static_cast<Box *>(ctx);
        try {
            body(*b->driver);
            return 0;
        } catch (...) {
            b->failure = std::current_exception();
            return EIO;
        }
    }
};

// ExpertLoadOperation (Infrastructure/Streaming/ExpertLoadOperation.swift:15-153): a shared handle
class ExpertLoadOperation {
public:
    ExpertLoadOperation() : h_(shrike_load_operation_create()) {
        if (!h_) throw Error(ENOMEM, "load operation");
    }
    ExpertLoadOperation(const ExpertLoadOperation &o) : h_(o.h_) { shrike_load_operation_retain(h_); }
    ExpertLoadOperation &operator=(const ExpertLoadOperation &o) {
        shrike_load_operation_retain(o.h_);
        shrike_load_operation_release(h_);
        h_ = o.h_;
        return *this;
    }
    ~ExpertLoadOperation() { shrike_load_operation_release(h_); }
    int state() const { return shrike_load_operation_state(h_); }
    void markInFlight() { check(shrike_load_operation_mark_in_flight(h_)); }
    void finish(int failure = 0) { check(shrike_load_operation_finish(h_, failure)); }
    void wait() { check(shrike_load_operation_wait(h_)); }
    bool wait(uint64_t untilNanos) { return shrike_load_operation_wait_until(h_, untilNanos) != 0; }
    uint64_t completedNanos() const { return shrike_load_operation_completed_nanos(h_); }
    shrike_load_operation *handle() const { return h_; }

private:
    shrike_load_operation *h_;
};

// ExpertIOScheduler (Infrastructure/Streaming/ExpertLoadOperation.swift:166-219) over the library's submission
// threads: a queued demand batch runs before any queued speculative one. The destructor runs what is queued,
// then joins the threads.
class ExpertIOScheduler {
public:
    enum class Priority { demand = SHRIKE_IO_DEMAND, speculative = SHRIKE_IO_SPECULATIVE };
    explicit ExpertIOScheduler(int workerCount = 4) {
        int err = 0;
        h_ = shrike_io_scheduler_create(workerCount, &err);
        if (!h_) throw Error(err, shrike_hip_last_error());
    }
    ~ExpertIOScheduler() { shrike_io_scheduler_destroy(h_); }
    ExpertIOScheduler(const ExpertIOScheduler &) = delete;
    ExpertIOScheduler &operator=(const ExpertIOScheduler &) = delete;
    void submit(std::function<void()> work, Priority priority = Priority::demand) {
        auto *boxed = new std::function<void()>(std::move(work));
        const int rc = shrike_io_scheduler_submit(h_, int(priority), &ExpertIOScheduler::run, boxed);
        if (rc != 0) {
            delete boxed;
            throw Error(rc, shrike_hip_last_error());
        }
    }
    void close() { shrike_io_scheduler_close(h_); }

private:
    static void run(void *context) {
        std::unique_ptr<std::function<void()>> work(static_cast<std::function<void()> *>(context));
        (*work)();
    }
    shrike_io_scheduler *h_;
};

// ExpertIOEventCoordinator + ExpertIOCompletionToken (Infrastructure/Streaming/ExpertIOEventCoordinator.swift:7-90)
using ExpertIOCompletionToken = shrike_io_completion_token;
class ExpertIOEventCoordinator {
public:
    static constexpr uint32_t statusWordCount = SHRIKE_IO_STATUS_WORDS;
    // statusWords: memory the GPU can read (pinned host memory) for the ring, or nullptr for words of its own
    explicit ExpertIOEventCoordinator(uint32_t *statusWords = nullptr, uint32_t wordCount = statusWordCount) {
        int err = 0;
        h_ = shrike_io_timeline_create(statusWords, wordCount, &err);
        if (!h_) throw Error(err, shrike_hip_last_error());
    }
    ~ExpertIOEventCoordinator() { shrike_io_timeline_destroy(h_); }
    ExpertIOEventCoordinator(const ExpertIOEventCoordinator &) = delete;
    ExpertIOEventCoordinator &operator=(const ExpertIOEventCoordinator &) = delete;
    ExpertIOCompletionToken reserve() {
        ExpertIOCompletionToken token;
        check(shrike_io_timeline_reserve(h_, &token));
        return token;
    }
    uint64_t publish(const ExpertIOCompletionToken &token, bool succeeded) { return shrike_io_timeline_publish(h_, &token, succeeded); }
    uint64_t signaledValue() { return shrike_io_timeline_published(h_); }

private:
    shrike_io_timeline *h_;
};

// RouterHostReadback (Runtime/Inference/RouterHostReadback.swift:8-63)
struct RouterHostReadback {
    static constexpr uint32_t tagBits = 16, valueMask = 0xffff, fixedWords = 2;
    int hitCount = 0, missCount = 0;
    std::vector<uint32_t> expertIDs;
    std::vector<uint16_t> weightBits;
    std::vector<uint32_t> hitPositions, missPositions, predictedIDs;
    static int wordCount(int topK) { return int(shrike_router_readback_word_count(uint32_t(topK))); }
    static uint32_t word(uint32_t tag, uint32_t value) { return shrike_router_readback_word(tag, value); }
    static uint32_t nextTag(uint32_t after) { return shrike_router_readback_next_tag(after); }
    static bool isComplete(const uint32_t *words, int topK, uint32_t tag) {
        return shrike_router_readback_is_complete(words, uint32_t(topK), tag) != 0;
    }
    static std::optional<RouterHostReadback> decode(const uint32_t *words, int topK, uint32_t tag) {
        shrike_router_readback r;
        if (!shrike_router_readback_decode(words, uint32_t(topK), tag, &r)) return std::nullopt;
        return from(r, topK);
    }
    // the runner's wait while the command still runs (RealForwardRunner.swift:3294-3310)
    static std::optional<RouterHostReadback> poll(const uint32_t *words, int topK, uint32_t tag, uint64_t timeoutNanos) {
        shrike_router_readback r;
        if (!shrike_router_readback_poll(words, uint32_t(topK), tag, shrike_monotonic_nanos() + timeoutNanos, &r)) return std::nullopt;
        return from(r, topK);
    }

private:
    static RouterHostReadback from(const shrike_router_readback &r, int topK) {
        RouterHostReadback out;
        out.hitCount = int(r.hit_count);
        out.missCount = int(r.miss_count);
        out.expertIDs.assign(r.expert_ids, r.expert_ids + topK);
        out.weightBits.assign(r.weight_bits, r.weight_bits + topK);
        out.hitPositions.assign(r.hit_positions, r.hit_positions + r.hit_count);
        out.missPositions.assign(r.miss_positions, r.miss_positions + r.miss_count);
        out.predictedIDs.assign(r.predicted_ids, r.predicted_ids + topK);
        return out;
    }
};

// CPUExpertFFN (Kernels/CPU/CPUExpertFFN.swift:10-140): the CPU expert kernel over host memory
struct CPUExpertFFN {
    static void gemv(const uint8_t *weights, const uint16_t *scales, const uint16_t *biases, const float *x, size_t rows, size_t n,
                     float *out) {
        shrike_int4_affine_gemv(weights, scales, biases, x, rows, n, out);
    }
    static size_t scratchFloats(uint32_t d, uint32_t f) { return shrike_cpu_expert_ffn_scratch_floats(d, f); }
    static void accumulate(const void *expert, const shrike_expert_offsets &offsets, const float *x, uint32_t d, uint32_t f,
                           float routeWeight, float *scratch, float *out) {
        check(shrike_cpu_expert_ffn_accumulate(expert, &offsets, x, d, f, routeWeight, scratch, out));
    }
};

// ExpertPrefetchRing (Runtime/Inference/ExpertPrefetchRing.swift:42-352)
class ExpertPrefetchRing {
public:
    using Drop = std::function<void(int layer, int expert, int cell)>;
    using Issue = std::function<ExpertLoadOperation(const std::vector<int> &experts, const std::vector<int> &cells)>;
    ExpertPrefetchRing(const std::vector<int> &cells, Drop drop) : drop_(std::move(drop)) {
        int err = 0;
        h_ = shrike_prefetch_ring_create(cells.data(), cells.size(),
                                         [](void *c, int layer, int expert, int cell) { static_cast<ExpertPrefetchRing *>(c)->drop_(layer, expert, cell); },
                                         this, &err);
        if (!h_) throw Error(err, "invalid prefetch ring geometry");
    }
    ~ExpertPrefetchRing() { shrike_prefetch_ring_destroy(h_); }
    ExpertPrefetchRing(const ExpertPrefetchRing &) = delete;
    ExpertPrefetchRing &operator=(const ExpertPrefetchRing &) = delete;
    void begin(int layer, const std::vector<int> &experts, const std::vector<int> &resident, const Issue &issue, bool deferred = false) {
        struct Box {
            const Issue *issue;
            std::exception_ptr failure;
            shrike_load_operation *handed;  // one reference that outlives the issue's own until the ring holds its
        } box{&issue, nullptr, nullptr};
        const int rc = shrike_prefetch_ring_begin(
            h_, layer, experts.data(), experts.size(), resident.data(), resident.size(), deferred,
            [](void *c, const int *e, const int *cells, size_t n, shrike_load_operation **out) -> int {
                Box *b = static_cast<Box *>(c);
                try {
                    ExpertLoadOperation op = (*b->issue)(std::vector<int>(e, e + n), std::vector<int>(cells, cells + n));
                    shrike_load_operation_retain(op.handle());
                    b->handed = *out = op.handle();
                    return 0;
                } catch (const PrefetchClaimRefused &) {
                    return SHRIKE_PREFETCH_CLAIM_REFUSED;
                } catch (...) {
                    b->failure = std::current_exception();
                    return EIO;
                }
            },
            &box);
        shrike_load_operation_release(box.handed);
        if (box.failure) std::rethrow_exception(box.failure);
        check(rc);
    }
    std::map<int, int> readyCells(int layer, const std::vector<int> &experts, uint64_t joinNanos = 0) {
        std::vector<int> e(experts.size() + 1), c(experts.size() + 1);
        const size_t n = shrike_prefetch_ring_ready_cells(h_, layer, experts.data(), experts.size(), joinNanos, e.data(), c.data());
        return zip(e, c, n);
    }
    void consume(int layer, const std::vector<int> &experts, const std::map<int, int> &freedCells) {
        std::vector<int> fe, fc;
        for (auto &kv : freedCells) {
            fe.push_back(kv.first);
            fc.push_back(kv.second);
        }
        shrike_prefetch_ring_consume(h_, layer, experts.data(), experts.size(), fe.data(), fc.data(), fe.size());
    }
    std::map<int, int> claimDemand(int layer, const std::vector<int> &experts) {
        std::vector<int> e(experts.size() + 1), c(experts.size() + 1);
        const size_t n = shrike_prefetch_ring_claim_demand(h_, layer, experts.data(), experts.size(), e.data(), c.data());
        return zip(e, c, n);
    }
    void attachDemand(int layer, const std::vector<int> &experts, const ExpertLoadOperation &operation) {
        shrike_prefetch_ring_attach_demand(h_, layer, experts.data(), experts.size(), operation.handle());
    }
    void unlease(int layer, const std::vector<int> &experts) { shrike_prefetch_ring_unlease(h_, layer, experts.data(), experts.size()); }
    void noteDemandSubmission() { shrike_prefetch_ring_note_demand_submission(h_); }
    bool noteHookFailure() { return shrike_prefetch_ring_note_hook_failure(h_) != 0; }
    shrike_prefetch_statistics statistics() const {
        shrike_prefetch_statistics st;
        shrike_prefetch_ring_statistics(h_, &st);
        return st;
    }
    int inFlightCount() const { return shrike_prefetch_ring_in_flight_count(h_); }
    int leasedCount() const { return shrike_prefetch_ring_leased_count(h_); }

private:
    static std::map<int, int> zip(const std::vector<int> &k, const std::vector<int> &v, size_t n) {
        std::map<int, int> out;
        for (size_t i = 0; i < n; ++i) out[k[i]] = v[i];
        return out;
    }
    shrike_prefetch_ring *h_;
    Drop drop_;
};

}  // namespace shrike
