// The reference's host-side unit tests, written against include/shrike.hpp the way the
// reference writes them against its Swift classes. No GPU call is made: budget ladder,
// grouping, sweep order, wave planner, slot cache, the packed-experts layout and the parallel reader run on the host. Exit code 0 = all passed.
#include <array>
#include <cmath>
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <optional>
#include <string>
#include <unistd.h>

#include "shrike.hpp"

using namespace shrike;

static int failures = 0;
#define EXPECT(cond)                                                      \
    do {                                                                  \
        if (!(cond)) {                                                    \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            ++failures;                                                   \
        }                                                                 \
    } while (0)

static shrike_token_expert_pair pair(uint32_t token, uint32_t expert, uint32_t rank, uint32_t bits) { return {token, expert, rank, bits}; }

// ExpertCacheBudgetTests.swift:20-29, :85-89, :117-153
static void budget() {
    EXPECT(RuntimeConfiguration::expertCacheSlots(1769472, 40) == 128);
    EXPECT(RuntimeConfiguration::expertCacheSlots(3342336, 40) == 64);
    EXPECT(RuntimeConfiguration::expertCacheSlots(1769472, 40, 11324620800LL) == 160);
    EXPECT(RuntimeConfiguration::parseBudgetBytes("8G") == int64_t(8) << 30);
    EXPECT(RuntimeConfiguration::parseBudgetBytes(" 4G ") == int64_t(4) << 30);
    EXPECT(RuntimeConfiguration::parseBudgetBytes("1.5G") == int64_t(1.5 * double(1 << 30)));
    for (const char *bad : {"", " ", "bogus", "G", "-2G", "0", "0G", "abcG", "2X", "2GG"}) EXPECT(!RuntimeConfiguration::parseBudgetBytes(bad));
    EXPECT(ExpertOffsets(2048, 512).strideBytes == 1769472);  // CPUExpertFFNTests.swift:56-67
}

// PrefillMoEGroupingTests.swift:5-53, :117-173
static void grouping() {
    std::vector<shrike_token_expert_pair> pairs = {
        pair(0, 3, 0, 10), pair(0, 1, 1, 11), pair(0, 4, 2, 12), pair(1, 1, 0, 13), pair(1, 3, 1, 14), pair(1, 2, 2, 15),
        pair(2, 4, 0, 16), pair(2, 3, 1, 17), pair(2, 1, 2, 18), pair(3, 5, 0, 19), pair(3, 1, 1, 20), pair(3, 4, 2, 21)};
    std::reverse(pairs.begin(), pairs.end());
    auto g = PrefillMoEGrouping::groupTokenExpertPairs(pairs, 4, 3, 6, 2);
    const uint32_t experts[12] = {1, 1, 1, 1, 2, 3, 3, 3, 4, 4, 4, 5};
    for (int i = 0; i < 12; ++i) EXPECT(g.sortedPairs[i].expert == experts[i]);
    EXPECT((g.perExpertOffsets == std::vector<uint32_t>{UINT32_MAX, 0, 4, 5, 8, 11}));
    EXPECT((g.perExpertCounts == std::vector<uint32_t>{0, 4, 1, 3, 3, 1}));
    EXPECT(g.groups.size() == 5 && g.tiles.size() == 3);
    EXPECT(g.tiles[1].group_start == 2 && g.tiles[1].group_count == 2 && g.tiles[1].pair_start == 5 && g.tiles[1].pair_count == 6);
    EXPECT(g.maxPairsPerExpert == 4 && g.maxPairsPerTile == 6 && g.maxLiveExpertsPerTile == 2);
    try {
        PrefillMoEGrouping::groupTokenExpertPairs({pair(0, 0, 0, 1), pair(0, 1, 0, 2)}, 1, 2, 2, 1);
        EXPECT(false);
    } catch (const GroupingError &e) {
        EXPECT(e.code == SHRIKE_GROUPING_DUPLICATE_TOKEN_RANK && e.values[0] == 0 && e.values[1] == 0);
    }
    try {
        PrefillMoEGrouping::groupTokenExpertPairs({pair(0, 0, 0, 1)}, 1, 1, 1, 17);
        EXPECT(false);
    } catch (const GroupingError &e) {
        EXPECT(e.code == SHRIKE_GROUPING_INVALID_TILE_EXPERT_COUNT && e.values[0] == 17);
    }
}

// PrefillMoEGroupingTests.swift:270-289, :205-246
static void sweepOrder() {
    std::vector<uint32_t> experts;
    std::vector<int64_t> rows, last;
    for (uint32_t id = 1; id <= 9; ++id) { experts.push_back(id); rows.push_back(1); last.push_back(9 + id); }
    for (uint32_t id = 100; id <= 102; ++id) { experts.push_back(id); rows.push_back(1); last.push_back(id - 100); }
    std::vector<uint8_t> resident(103, 0);
    for (int id = 1; id <= 9; ++id) resident[id] = 1;
    auto order = PrefillSweepOrder::residentFirstBalanced(experts, rows, last, resident, 20, 8);
    EXPECT((order == std::vector<uint32_t>{1, 2, 3, 4, 5, 6, 7, 8, 100, 101, 102, 9}));
    auto keys = PrefillSweepOrder::expertSortKeys({3, 8, 5}, 9);
    EXPECT(keys[3] == 0 && keys[8] == 1 && keys[5] == 2 && keys[0] == 3 && keys[7] == 3);
}

// PrefillGroupedRoutedMoETests+Execution.swift:382-432, :535-577
static void wavePlanner() {
    const std::vector<shrike_expert_pair_range> ranges = {{0, 0, 40}, {1, 40, 32}, {2, 72, 5}, {3, 77, 3}};
    auto one = PrefillGroupedRoutedMoE::planExpertWaves(ranges, {0, 1, 2, 3}, 512);
    EXPECT(one.size() == 1 && one[0].paddedRows == 256 && one[0].blocks.size() == 4);
    EXPECT(one[0].blocks[2].slot == 2 && one[0].blocks[2].pair_start == 72 && one[0].blocks[2].rows == 5 && one[0].blocks[2].staging_row == 128);
    EXPECT((PrefillGroupedRoutedMoE::rowTileTable(one[0]) == std::vector<uint32_t>{0, 1, 2, 3}));
    auto tailed = PrefillGroupedRoutedMoE::planExpertWaves(ranges, {0, 1, 2, 3}, 512, 64, 32);
    EXPECT(tailed.size() == 1 && tailed[0].paddedRows == 160 && tailed[0].tailRows == 96);
    auto longExpert = PrefillGroupedRoutedMoE::planExpertWaves({{2, 0, 600}}, {0, 1, 2, 3}, 512);
    EXPECT(longExpert.size() == 2 && longExpert[1].blocks[0].pair_start == 512 && longExpert[1].blocks[0].rows == 88 && longExpert[1].paddedRows == 128);
    try {
        PrefillGroupedRoutedMoE::planExpertWaves(ranges, {0, 1, 2, 3}, 96);
        EXPECT(false);
    } catch (const Error &e) {
        EXPECT(e.code == EINVAL);
    }
}

// PreadExpertStreamerTests+CachePlanning.swift:130-154, :225-270, :320-341
// PreadExpertStreamerTests+Landing.swift: aSwapThenAnEvictionOfTheSameSlotPublishesEmptyOnceAtTheCell,
// aPredictionThePoolHoldsRefusesTheBatch and anOverflowSlotIsAVictimOfThePoolLoadingAtItsCell
static void landings() {
    const auto word = [](uint32_t state, uint32_t cell) { return uint64_t(state) << 32 | cell; };
    {
        CellArena arena(4);
        SlotCache c(arena, 2, 4, 0);
        auto warm = c.planExpertsCached({0, 2});
        c.markPlanMissesResident(warm);
        const int64_t ring = 2;
        c.claimPrefetch({1}, {ring});
        EXPECT(c.completeLanding(1, ring));
        EXPECT(c.residencyEntry(1) == word(SHRIKE_RESIDENCY_RESIDENT, 2));
        auto swap = c.planExpertsCachedIfPossible({0, 1}, 0, {}, nullptr, -1, {}, {1});
        EXPECT(swap && swap->hits == 2 && swap->misses.empty());
        EXPECT(swap->assignedSlots == (std::vector<int32_t>{0, 1}));
        EXPECT(swap->freedCells == (std::map<int32_t, uint32_t>{{1, 1}}));
        EXPECT(swap->assignedGenerations == (std::vector<uint64_t>{1, 3}));
        EXPECT(swap->assignedCells == (std::vector<uint32_t>{0, 2}));
        EXPECT(arena.cellGeneration(1) == 4 && arena.cellGeneration(2) == 3);
        EXPECT(c.residencyEntry(2) == word(SHRIKE_RESIDENCY_EMPTY, 0xffffffffu));
        auto evict = c.planExpertsCached({3});
        EXPECT(evict.assignedSlots == (std::vector<int32_t>{1}) && evict.assignedGenerations == (std::vector<uint64_t>{5}));
        EXPECT(c.residencyEntry(3) == word(SHRIKE_RESIDENCY_LOADING, 2));
        EXPECT(c.ownsCell(2) && !c.ownsCell(1) && c.slotCell(1) == 2);
    }
    {
        CellArena arena(6);
        SlotCache c(arena, 4, 4, 0);
        auto warm = c.planExpertsCached({1});
        c.markPlanMissesResident(warm);
        bool refused = false;
        try {
            c.claimPrefetch({3, 1}, {4, 5});
        } catch (const PrefetchClaimRefused &r) {
            refused = r.expert == 1 && r.cell == 5;
        }
        EXPECT(refused);
        EXPECT(c.residencyEntry(3) == word(SHRIKE_RESIDENCY_EMPTY, 0xffffffffu));
        EXPECT(c.claimLanding(3, 4));
        bool owned = false;
        try {
            c.claimPrefetch({2}, {0});
        } catch (const Error &) {
            owned = true;
        }
        EXPECT(owned);
    }
    {
        CellArena arena(4);
        SlotCache c(arena, 2, 4, 0);
        auto warm = c.planExpertsCached({0, 1});
        c.markPlanMissesResident(warm);
        EXPECT(!c.reserveOverflowSlot(2, {0, 1}));
        const auto cell = c.reserveOverflowSlot(2, {0, 5});
        EXPECT(cell && *cell == 1);
        EXPECT(c.claimLanding(3, 2));
        c.finishAgreedReads({3, 2}, {2, int64_t(*cell)}, true);
        EXPECT(c.residencyEntry(3) == word(SHRIKE_RESIDENCY_RESIDENT, 2));
        EXPECT(c.residencyEntry(2) == word(SHRIKE_RESIDENCY_RESIDENT, *cell));
        EXPECT(c.statistics().read_operations == 4);
    }
}

// ExpertLoadOperation.swift:166-219: queued demand work runs ahead of queued speculative work
static void ioScheduler() {
    std::vector<int> order;
    std::mutex guard;
    {
        std::mutex gate;
        gate.lock();
        ExpertIOScheduler scheduler(1);
        scheduler.submit([&] { std::lock_guard<std::mutex> wait(gate); });  // holds the only worker while the queues fill
        for (int i = 0; i < 3; ++i)
            scheduler.submit([&, i] { std::lock_guard<std::mutex> g(guard); order.push_back(10 + i); }, ExpertIOScheduler::Priority::speculative);
        for (int i = 0; i < 3; ++i)
            scheduler.submit([&, i] { std::lock_guard<std::mutex> g(guard); order.push_back(i); });
        gate.unlock();
    }  // the destructor drains the queues
    EXPECT(order == (std::vector<int>{0, 1, 2, 10, 11, 12}));
}

// ExpertLoadOperationTests.swift:95-150: the timeline holds an out-of-order completion, a failure is terminal,
// status words recycle after one ring
static void ioCoordinator() {
    {
        ExpertIOEventCoordinator coordinator;
        auto first = coordinator.reserve(), second = coordinator.reserve();
        coordinator.publish(second, true);
        EXPECT(*second.status == 1 && coordinator.signaledValue() == 0);
        coordinator.publish(first, true);
        EXPECT(coordinator.signaledValue() == second.value && first.value != second.value);
    }
    {
        ExpertIOEventCoordinator coordinator;
        auto token = coordinator.reserve();
        coordinator.publish(token, false);
        EXPECT(*token.status == 2 && coordinator.signaledValue() == token.value);
    }
    {
        ExpertIOEventCoordinator coordinator;
        auto first = coordinator.reserve();
        for (uint32_t i = 1; i < ExpertIOEventCoordinator::statusWordCount; ++i) coordinator.publish(coordinator.reserve(), true);
        coordinator.publish(first, false);
        auto recycled = coordinator.reserve();
        EXPECT(recycled.value == first.value + ExpertIOEventCoordinator::statusWordCount);
        EXPECT(recycled.status == first.status && *recycled.status == 0);
        coordinator.publish(recycled, true);
        EXPECT(coordinator.signaledValue() == recycled.value);
    }
}

// RouterHostReadbackTests.swift:18-91
static void routerReadback() {
    const int topK = 4;
    auto words = [&](uint32_t tag, uint32_t hits = 3, uint32_t misses = 1) {
        const uint32_t values[] = {hits, misses, 5, 9, 200, 3, 0x3c00, 0x3800, 0x3400, 0x3000, 0, 2, 3, 0, 1, 0, 0, 0, 1, 2, 3, 4};
        std::vector<uint32_t> out;
        for (uint32_t v : values) out.push_back(RouterHostReadback::word(tag, v));
        return out;
    };
    EXPECT(RouterHostReadback::wordCount(4) == 22 && RouterHostReadback::wordCount(8) == 42);
    auto w = words(7);
    auto r = RouterHostReadback::decode(w.data(), topK, 7);
    EXPECT(r && r->hitCount == 3 && r->missCount == 1 && (r->expertIDs == std::vector<uint32_t>{5, 9, 200, 3}));
    EXPECT(r && (r->weightBits == std::vector<uint16_t>{0x3c00, 0x3800, 0x3400, 0x3000}) && (r->hitPositions == std::vector<uint32_t>{0, 2, 3}));
    EXPECT(r && (r->missPositions == std::vector<uint32_t>{1}) && (r->predictedIDs == std::vector<uint32_t>{1, 2, 3, 4}));
    w.back() = RouterHostReadback::word(6, 4);
    EXPECT(!RouterHostReadback::isComplete(w.data(), topK, 7) && !RouterHostReadback::decode(w.data(), topK, 7));
    std::vector<uint32_t> zeroed(22, 0u);
    EXPECT(!RouterHostReadback::isComplete(zeroed.data(), topK, 1));
    auto clamped = words(3, 9, 9);
    auto c = RouterHostReadback::decode(clamped.data(), topK, 3);
    EXPECT(c && c->hitCount == 4 && c->missCount == 4 && c->hitPositions.size() == 4);
    EXPECT(RouterHostReadback::nextTag(0) == 1 && RouterHostReadback::nextTag(5) == 6 && RouterHostReadback::nextTag(0xffff) == 1);
    EXPECT(!RouterHostReadback::poll(zeroed.data(), topK, 1, 1000000));
}

// CPUExpertFFNTests.swift:56-67 (the blob's size) and the closed form of MoEFusedFFNTests: codes 1, scale 1, bias 0
// make every projection a plain sum
static void cpuExpertFFN() {
    const uint32_t d = 128, f = 64;
    ExpertOffsets off(d, f, 4);
    std::vector<uint8_t> blob(off.strideBytes, 0);
    auto fill = [&](uint32_t w_off, uint32_t s_off, uint32_t rows, uint32_t n) {
        for (uint32_t i = 0; i < rows * n / 2; ++i) blob[w_off + i] = 0x11;
        for (uint32_t i = 0; i < rows * n / 64; ++i) {
            blob[s_off + 2 * i] = 0x80;  // bf16 1.0 = 0x3f80
            blob[s_off + 2 * i + 1] = 0x3f;
        }
    };
    fill(off.gate_w_off, off.gate_s_off, f, d);
    fill(off.up_w_off, off.up_s_off, f, d);
    fill(off.down_w_off, off.down_s_off, d, f);
    std::vector<float> x(d, 1.0f / d), out(d, 1.0f), scratch(CPUExpertFFN::scratchFloats(d, f));
    CPUExpertFFN::accumulate(blob.data(), off, x.data(), d, f, 0.5f, scratch.data(), out.data());
    // gate = up = 1, act = silu(1) = 1 / (1 + e^-1), down = f * act, out = 1 + 0.5 * that
    const float want = 1.0f + 0.5f * float(f) * (1.0f / (1.0f + std::exp(-1.0f)));
    for (float v : out) EXPECT(std::fabs(v - want) < 1e-4f);
}

static void slotCache() {
    {
        SlotCache c(4, 8);
        auto warm = c.planExpertsCached({0, 1});
        c.markPlanMissesResident(warm);
        auto plan = c.planExpertsCached({0, 2}, 0, {0, 1});
        EXPECT((plan.assignedSlots == std::vector<int32_t>{0, 2}) && plan.hits == 1 && (plan.misses == std::vector<uint32_t>{1}));
    }
    {
        SlotCache c(2, 8);
        for (auto experts : {std::vector<int32_t>{0, 1}, {0, 2}, {0, 1}}) {
            auto p = c.planExpertsCached(experts);
            c.markPlanMissesResident(p);
        }
        auto s = c.statistics(1000);
        EXPECT(s.plans == 3 && s.requested_experts == 6 && s.hits == 2 && s.misses == 4 && s.evictions == 2 && s.reloads == 1);
        EXPECT(s.read_operations == 4 && s.bytes_read == 4000 && s.load_batches == 3 && s.loading_slots == 0);
    }
    {
        SlotCache c(2, 8);
        auto warm = c.planExpertsCached({0, 1});
        c.markPlanMissesResident(warm);
        auto resident = c.planExpertsCached({0, 1});
        c.pin(resident);
        EXPECT(c.statistics().pinned_slots == 2 && !c.planExpertsCachedIfPossible({2}));
        c.unpin(resident);
        auto dropped = c.planExpertsCached({2, 3});
        EXPECT(dropped.misses.size() == 2 && c.statistics().loading_slots == 2 && !c.planExpertsCachedIfPossible({0}));
        c.abandonExpertCachePlan(dropped);
        EXPECT(c.statistics().loading_slots == 0);
        EXPECT((c.residencyEntry(2) >> 32) == SHRIKE_RESIDENCY_EMPTY);
    }
}

// PackedExpertsLayoutTests.swift:10-90 (the toy layout) and ParallelExpertReaderTests.swift:36-58, :132-158
static void layoutAndReader() {
    const char *tensors = "{\"gate\": {\"offset\": 0, \"size\": 4096, \"dtype\": \"U32\", \"shape\": [64, 64], \"bits\": 4},"
                          " \"gate_scales\": {\"offset\": 4096, \"size\": 256, \"dtype\": \"BF16\", \"shape\": [64, 1]}}";
    const std::string json = std::string("{\"expertStride\": 16384, \"numLayers\": 1, \"expertsPerLayer\": 2, \"layers\": [{\"layer\": 0,"
        " \"file\": \"layer_00.bin\", \"experts\": [{\"expert\": 0, \"offset\": 0, \"size\": 16384, \"tensors\": ") + tensors
        + "}, {\"expert\": 1, \"physicalRank\": 1, \"offset\": 16384, \"size\": 16384, \"tensors\": " + tensors + "}]}]}";
    auto layout = PackedExpertsLayout::decode(json);
    EXPECT(layout.expertStride() == 16384 && layout.numLayers() == 1 && layout.expertsPerLayer() == 2);
    EXPECT(layout.file(0) == "layer_00.bin");
    EXPECT(layout.expert(0, 0).offset == 0 && layout.expert(0, 0).size == 16384);
    EXPECT(layout.subTensor(0, 0, "gate")->offset == 0 && layout.subTensor(0, 0, "gate_scales")->offset == 4096);
    EXPECT(layout.expert(0, 1).offset == 16384 && layout.expert(0, 1).expert == 1);
    EXPECT(!layout.subTensor(0, 0, "down"));
    EXPECT(layout.routedExpertOffsets(0).gate_s_off == 4096 && layout.routedExpertOffsets(0).down_w_off == 0);
    bool threw = false;
    try { layout.expert(0, 2); } catch (const Error &e) { threw = std::string(e.what()).find("layer 0 has 2 experts; expert 2 is out of range") != std::string::npos; }
    EXPECT(threw);
    threw = false;
    try { PackedExpertsLayout::decode("{\"expertStride\": 100, \"numLayers\": 1, \"expertsPerLayer\": 1, \"layers\": []}"); }
    catch (const Error &e) { threw = e.code == EINVAL && std::string(e.what()).find("invalid dimensions or stride") != std::string::npos; }
    EXPECT(threw);

    // a file of 64 blocks, block e filled with e % 251; out-of-order ids with a repeat
    const size_t stride = 4096;
    char path[] = "/tmp/shrike_reader_XXXXXX";
    const int fd = mkstemp(path);
    EXPECT(fd >= 0);
    std::vector<unsigned char> block(stride);
    for (int e = 0; e < 64; ++e) {
        std::fill(block.begin(), block.end(), static_cast<unsigned char>(e % 251));
        EXPECT(write(fd, block.data(), stride) == ssize_t(stride));
    }
    close(fd);
    {
        ParallelExpertReader reader(path, stride, 4, 2);
        EXPECT(reader.threadCount() == 4 && reader.batchDepth() == 2);
        const std::vector<uint32_t> wanted = {63, 0, 17, 17, 40, 5, 62, 1};
        std::vector<std::vector<unsigned char>> buffers(wanted.size(), std::vector<unsigned char>(stride));
        std::vector<void *> into;
        for (auto &b : buffers) into.push_back(b.data());
        reader.fetch(wanted, into);
        for (size_t i = 0; i < wanted.size(); ++i) EXPECT(buffers[i][0] == wanted[i] % 251 && buffers[i][stride - 1] == wanted[i] % 251);
        reader.fetch(std::vector<uint32_t>{}, {});
        threw = false;
        try { reader.fetch(std::vector<uint32_t>{99}, {buffers[0].data()}); } catch (const ParallelExpertReader::Failure &e) { threw = e.code == EIO; }
        EXPECT(threw);
        EXPECT(ParallelExpertReader(path, stride, 0, 0).threadCount() == 1);
        EXPECT(ParallelExpertReader(path, stride, 999, 9).threadCount() == 16);
    }
    unlink(path);
    threw = false;
    try { ParallelExpertReader missing("/nonexistent/shrike/experts.bin", 4096); } catch (const ParallelExpertReader::Failure &e) { threw = e.code == ENOENT; }
    EXPECT(threw);
}

// PrefillRoutedTileSchedulerTests / PrefillRoutedTileSequencerTests / ExpertPrefetchRingTests, a few cases each
struct RecordingDriver : PrefillRoutedTileDriver {
    std::vector<std::string> calls;
    std::vector<int> open;
    std::vector<std::vector<int>> pending;
    int failingEncode = -1;
    std::vector<int> slots(int tile) { return {2 * tile, 2 * tile + 1}; }
    int openBatchTiles() override { return int(open.size()); }
    size_t openBatchSlotCount() override { return 2 * open.size(); }
    int pendingDepth() override { return int(pending.size()); }
    size_t pendingAssignedSlotCount() override {
        size_t n = 0;
        for (auto &b : pending) n += b.size();
        return n;
    }
    bool plan(int tile, std::optional<int> avoiding) override {
        calls.push_back("plan" + std::to_string(tile) + (avoiding ? "/" + std::to_string(*avoiding) : ""));
        return true;
    }
    void begin(int tile) override { calls.push_back("begin" + std::to_string(tile)); }
    void abandonPlan(int tile) override { calls.push_back("abandonPlan" + std::to_string(tile)); }
    void encode(int tile) override {
        calls.push_back("encode" + std::to_string(tile));
        if (tile == failingEncode) throw std::runtime_error("encode failed");
        open.push_back(tile);
    }
    void commitOpenBatch() override {
        if (open.empty()) return;
        calls.push_back("commit");
        std::vector<int> all;
        for (int t : open)
            for (int s : slots(t)) all.push_back(s);
        pending.push_back(all);
        open.clear();
    }
    void drainOldestBatch() override {
        calls.push_back("drain");
        if (!pending.empty()) pending.erase(pending.begin());
    }
    void abandonBegunFetches() override { calls.push_back("abandonBegun"); }
};

static void tileLoopAndRing() {
    PrefillRoutedTileSchedulerConfig def;
    auto fit = def.fitting(8);
    EXPECT(fit && fit->max_pending_depth == 1 && fit->tile_experts == 4 && fit->tiles_per_command_buffer == 1);
    EXPECT(!def.fitting(1));
    EXPECT(PrefillRoutedTileSchedulerConfig(2, 4).fitsSlotBudget(16) && !PrefillRoutedTileSchedulerConfig(2, 8).fitsSlotBudget(16));
    PrefillRoutedTileScheduler sch{PrefillRoutedTileSchedulerConfig(2, 4)};
    EXPECT(sch.decide(false, 0, false) == SHRIKE_TILE_ISSUE_WITHOUT_PENDING);
    EXPECT(sch.decide(true, 8, true, 2) == SHRIKE_TILE_PREFETCH_NEXT);
    EXPECT(sch.decide(true, 2, true, 3) == SHRIKE_TILE_DRAIN_MAX_DEPTH);
    {
        RecordingDriver d;
        PrefillRoutedTileSequencer{PrefillRoutedTileScheduler{PrefillRoutedTileSchedulerConfig(2, 8, 1, 1)}}.run(3, d);
        const std::vector<std::string> want = {"plan0", "begin0", "plan1/0", "begin1", "encode0", "commit", "plan2/1", "begin2",
                                               "encode1", "commit", "encode2", "commit", "drain", "drain", "drain"};
        EXPECT(d.calls == want);
    }
    {
        RecordingDriver d;
        d.failingEncode = 0;
        bool thrown = false;
        try {
            PrefillRoutedTileSequencer{PrefillRoutedTileScheduler{PrefillRoutedTileSchedulerConfig(2, 8, 1, 1)}}.run(3, d);
        } catch (const std::runtime_error &e) {
            thrown = std::string(e.what()) == "encode failed";
        }
        const std::vector<std::string> want = {"plan0", "begin0", "plan1/0", "begin1", "encode0", "abandonBegun"};
        EXPECT(thrown && d.calls == want);
    }
    {
        std::vector<std::array<int, 3>> drops;
        ExpertPrefetchRing ring({10, 11, 12, 13}, [&](int l, int e, int c) { drops.push_back({l, e, c}); });
        std::vector<std::vector<int>> issued;
        ExpertLoadOperation first;
        ring.begin(3, {7, 9, 11}, {}, [&](const std::vector<int> &e, const std::vector<int> &) { issued.push_back(e); return first; });
        EXPECT(issued.size() == 1 && issued[0] == std::vector<int>{7} && ring.inFlightCount() == 1);
        ring.begin(4, {1, 2}, {}, [&](const std::vector<int> &e, const std::vector<int> &) { issued.push_back(e); return ExpertLoadOperation(); });
        EXPECT(issued.size() == 1 && ring.statistics().issued == 1);
        first.markInFlight();
        first.finish();
        ring.begin(4, {1, 2}, {}, [&](const std::vector<int> &e, const std::vector<int> &) { issued.push_back(e); return ExpertLoadOperation(); });
        EXPECT(issued.size() == 2 && issued[1] == std::vector<int>{1});
        EXPECT(ring.statistics().issued == 2 && ring.statistics().reclaimed == 1 && drops.size() == 1 && drops[0][1] == 7);
        // a refused claim is counted, an issue that throws rolls the slots back
        ExpertPrefetchRing other({20, 21}, [](int, int, int) {});
        other.begin(2, {1, 2}, {}, [](const std::vector<int> &e, const std::vector<int> &c) -> ExpertLoadOperation { throw PrefetchClaimRefused{e[0], c[0]}; });
        EXPECT(other.statistics().refused == 2 && other.inFlightCount() == 0);
        bool thrown = false;
        try {
            other.begin(2, {1}, {}, [](const std::vector<int> &, const std::vector<int> &) -> ExpertLoadOperation { throw std::runtime_error("reader refused"); });
        } catch (const std::runtime_error &) {
            thrown = true;
        }
        EXPECT(thrown && other.inFlightCount() == 0);
        ExpertLoadOperation op;
        other.begin(2, {1}, {}, [&](const std::vector<int> &, const std::vector<int> &) { return op; });
        op.finish();
        auto ready = other.readyCells(2, {1});
        EXPECT(ready.size() == 1 && ready[1] == 20 && other.leasedCount() == 1);
        other.consume(2, {1}, {{1, 77}});
        EXPECT(other.statistics().adopted == 1 && other.leasedCount() == 0);
        auto claimed = other.claimDemand(5, {4, 6, 8});
        EXPECT(claimed.size() == 2 && claimed[4] == 77 && claimed[6] == 21);
    }
}

int main() {
    tileLoopAndRing();
    layoutAndReader();
    budget();
    grouping();
    sweepOrder();
    wavePlanner();
    slotCache();
    landings();
    ioScheduler();
    ioCoordinator();
    routerReadback();
    cpuExpertFFN();
    std::printf(failures ? "%d checks failed\n" : "all host checks passed\n", failures);
    return failures ? 1 : 0;
}
