// The slot cache's bookkeeping: which expert sits in which slot of the HBM pool, which
// slot a miss may take, and the residency words the kernels classify against
// (PreadExpertStreamer.swift:405-543, :676-767, :1085-1148), the landings a prefetch ring
// claims in cells outside the pool and the overflow slots of a decode route (:815-1018),
// and the arena-wide cell generations (ExpertCellArena.swift:95-104). No device calls: the
// owner mirrors the drained publications into the pool's device table.
#include <algorithm>
#include <atomic>
#include <cmath>
#include <memory>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "../../include/shrike_host.h"
#include "host_common.h"

using shrike::set_error;

namespace {
enum : uint8_t { kEmpty = 0, kLoading = 1, kResident = 2 };
}

// ExpertCellArena's numbering and generations: one clock for every cell, so a generation
// never repeats across the cells a slot may come to hold.
struct shrike_cell_arena {
    uint32_t cell_count = 0;
    std::unique_ptr<std::atomic<uint64_t>[]> generations;
    std::atomic<uint64_t> clock{0};

    uint64_t generation(uint32_t cell) const { return generations[cell].load(std::memory_order_relaxed); }
    uint64_t bump(uint32_t cell) {  // bumpCellGeneration, ExpertCellArena.swift:99-104
        const uint64_t g = clock.fetch_add(1, std::memory_order_relaxed) + 1;
        generations[cell].store(g, std::memory_order_relaxed);
        return g;
    }
};

namespace {
shrike_cell_arena *make_arena(uint32_t cell_count) {
    auto *a = new (std::nothrow) shrike_cell_arena();
    if (!a) return nullptr;
    a->cell_count = cell_count;
    a->generations.reset(new (std::nothrow) std::atomic<uint64_t>[cell_count]);
    if (!a->generations) {
        delete a;
        return nullptr;
    }
    for (uint32_t i = 0; i < cell_count; ++i) a->generations[i].store(0, std::memory_order_relaxed);
    return a;
}

struct Landing {  // PreadExpertStreamer.swift:198-202
    uint32_t cell;
    bool resident;
    uint64_t generation;
};
}  // namespace

struct shrike_slot_cache {
    uint32_t slot_count, experts_per_layer;
    shrike_cell_arena *arena = nullptr;
    bool owns_arena = false;
    bool slru;
    int64_t protected_capacity;
    std::mutex lock;
    std::vector<int32_t> slot_expert;
    std::vector<int64_t> slot_last_use;
    std::vector<uint8_t> slot_state, slot_protected, reserved;
    std::vector<int64_t> slot_pins;
    std::vector<int64_t> use_count, load_count;
    std::vector<uint32_t> slot_cell;  // the arena cell behind each slot; a landing's swap changes it
    std::vector<uint8_t> overflow_probation;
    std::unordered_map<int32_t, Landing> landings;
    std::vector<int32_t> victims;
    std::vector<uint64_t> words;
    std::vector<uint8_t> dirty;
    std::vector<uint32_t> dirty_order;
    int64_t use_clock = 0;
    int64_t protected_count = 0;
    shrike_streaming_statistics stats{};

    ~shrike_slot_cache() {
        if (owns_arena) delete arena;
    }

    uint32_t cell(int32_t slot) const { return slot_cell[size_t(slot)]; }  // cellIndexUnlocked
    uint64_t generation_of(int32_t slot) const { return arena->generation(cell(slot)); }
    bool holds(int32_t expert) const {  // slotExpert.contains(expert)
        return std::find(slot_expert.begin(), slot_expert.end(), expert) != slot_expert.end();
    }
    int32_t slot_of_cell(uint32_t c) const {  // slotIndexUnlocked(cell:)
        for (uint32_t s = 0; s < slot_count; ++s)
            if (slot_cell[s] == c) return int32_t(s);
        return -1;
    }
    void demote(int32_t slot) {  // demoteIfProtected, :722-726
        if (!slot_protected[size_t(slot)]) return;
        slot_protected[size_t(slot)] = 0;
        --protected_count;
    }
    void reserve_loading() {
        std::fill(reserved.begin(), reserved.end(), 0);
        for (uint32_t s = 0; s < slot_count; ++s)
            if (slot_state[s] == kLoading) reserved[s] = 1;
    }
    void record_batch(uint64_t count, uint64_t elapsed_nanos, uint64_t fetch_nanos) {  // recordLoadBatchUnlocked, :1158-1168
        stats.read_operations += count;
        ++stats.load_batches;
        stats.total_load_nanos += elapsed_nanos;
        stats.fetch_nanos += fetch_nanos;
        stats.maximum_load_nanos = std::max(stats.maximum_load_nanos, elapsed_nanos);
        uint64_t bound = 125000;  // latencyBucketIndex, :1181-1188
        int bucket = 16;
        for (int index = 0; index < 16; ++index) {
            if (elapsed_nanos <= bound) {
                bucket = index;
                break;
            }
            bound *= 2;
        }
        ++stats.latency_histogram[bucket];
    }
    void record_expert_load(int32_t e) {  // recordExpertLoadsUnlocked, :1170-1179
        if (e < 0 || size_t(e) >= load_count.size()) return;
        if (load_count[size_t(e)] > 0) ++stats.reloads;
        ++load_count[size_t(e)];
    }

    // PreadExpertStreamer.swift:1143-1148: an empty entry names the sentinel cell
    void publish(int32_t expert, uint32_t cell_index, uint32_t state) {
        if (expert < 0 || uint32_t(expert) >= experts_per_layer) return;
        const uint32_t slot = state == kEmpty ? 0xffffffffu : cell_index;
        words[size_t(expert)] = uint64_t(state) << 32 | slot;
        if (!dirty[size_t(expert)]) {
            dirty[size_t(expert)] = 1;
            dirty_order.push_back(uint32_t(expert));
        }
    }

    // shouldEvictSlot, :728-742
    bool evict_before(int32_t lhs, int32_t rhs) const {
        const int32_t le = slot_expert[size_t(lhs)], re = slot_expert[size_t(rhs)];
        if (le < 0 || re < 0) return le < re;
        if (slru) {
            if (slot_protected[size_t(lhs)] != slot_protected[size_t(rhs)]) return !slot_protected[size_t(lhs)];
            return slot_last_use[size_t(lhs)] < slot_last_use[size_t(rhs)];
        }
        const int64_t lc = size_t(le) < use_count.size() ? use_count[size_t(le)] : 0;
        const int64_t rc = size_t(re) < use_count.size() ? use_count[size_t(re)] : 0;
        if (lc != rc) return lc < rc;
        return slot_last_use[size_t(lhs)] < slot_last_use[size_t(rhs)];
    }

    // selectVictimSlots, :676-705: the best miss_count victims in comparator order, ties to
    // the lower slot
    bool select_victims(uint32_t miss_count, const uint8_t *protected_experts, uint32_t protected_len) {
        uint32_t victim_count = 0, eligible = 0;
        for (int32_t slot = 0; slot < int32_t(slot_count); ++slot) {
            if (reserved[size_t(slot)] || slot_state[size_t(slot)] == kLoading || slot_pins[size_t(slot)] != 0) continue;
            const int32_t e = slot_expert[size_t(slot)];
            if (protected_experts && e >= 0 && uint32_t(e) < protected_len && protected_experts[e]) continue;
            ++eligible;
            if (victim_count < miss_count) {
                uint32_t at = victim_count;
                while (at > 0 && evict_before(slot, victims[at - 1])) {
                    victims[at] = victims[at - 1];
                    --at;
                }
                victims[at] = slot;
                ++victim_count;
            } else if (victim_count > 0 && evict_before(slot, victims[victim_count - 1])) {
                uint32_t at = victim_count - 1;
                while (at > 0 && evict_before(slot, victims[at - 1])) {
                    victims[at] = victims[at - 1];
                    --at;
                }
                victims[at] = slot;
            }
        }
        return miss_count <= eligible;
    }

    // promoteToProtected, :708-720
    void promote(int32_t slot, int64_t clock) {
        slot_protected[size_t(slot)] = 1;
        ++protected_count;
        if (protected_count <= protected_capacity) return;
        int32_t oldest = -1;
        for (int32_t c = 0; c < int32_t(slot_count); ++c) {
            if (!slot_protected[size_t(c)] || c == slot) continue;
            if (oldest < 0 || slot_last_use[size_t(c)] < slot_last_use[size_t(oldest)]) oldest = c;
        }
        if (oldest < 0) return;
        slot_protected[size_t(oldest)] = 0;
        --protected_count;
        slot_last_use[size_t(oldest)] = clock;
    }

    uint32_t count_state(uint8_t state) const {
        return uint32_t(std::count(slot_state.begin(), slot_state.end(), state));
    }
};

extern "C" {

shrike_cell_arena *shrike_cell_arena_create(uint32_t cell_count, int *out_errno) {
    if (out_errno) *out_errno = 0;
    if (cell_count == 0) {  // ExpertCellArena.swift:32-35
        set_error("invalid expert cell arena geometry: 0 cells");
        if (out_errno) *out_errno = EINVAL;
        return nullptr;
    }
    shrike_cell_arena *a = make_arena(cell_count);
    if (!a) {
        set_error("cell arena allocation failed");
        if (out_errno) *out_errno = ENOMEM;
    }
    return a;
}

void shrike_cell_arena_destroy(shrike_cell_arena *arena) { delete arena; }

uint32_t shrike_cell_arena_cell_count(const shrike_cell_arena *arena) { return arena ? arena->cell_count : 0; }

uint64_t shrike_cell_arena_generation(const shrike_cell_arena *arena, uint32_t cell) {
    return arena && cell < arena->cell_count ? arena->generation(cell) : 0;
}

static shrike_slot_cache *create_cache(shrike_cell_arena *arena, bool owns_arena, uint32_t slot_count,
                                       uint32_t experts_per_layer, uint32_t first_cell, int policy,
                                       double slru_protected_share, int *out_errno) {
    auto *c = new (std::nothrow) shrike_slot_cache();
    if (!c) {
        if (owns_arena) delete arena;
        set_error("slot cache allocation failed");
        if (out_errno) *out_errno = ENOMEM;
        return nullptr;
    }
    c->slot_count = slot_count;
    c->experts_per_layer = experts_per_layer;
    c->arena = arena;
    c->owns_arena = owns_arena;
    c->slru = policy == SHRIKE_EVICT_SLRU;
    // ExpertEvictionPolicy.protectedCapacity, Model.swift:26-33
    c->protected_capacity = c->slru ? std::max<int64_t>(1, int64_t(std::round(slru_protected_share * double(slot_count)))) : 0;
    const size_t n = slot_count, e = std::max<uint32_t>(1, experts_per_layer);
    c->slot_expert.assign(n, -1);
    c->slot_last_use.assign(n, 0);
    c->slot_state.assign(n, kEmpty);
    c->slot_protected.assign(n, 0);
    c->reserved.assign(n, 0);
    c->slot_pins.assign(n, 0);
    c->use_count.assign(e, 0);
    c->load_count.assign(e, 0);
    c->slot_cell.resize(n);
    for (uint32_t s = 0; s < slot_count; ++s) c->slot_cell[s] = first_cell + s;
    c->overflow_probation.assign(n, 0);
    c->victims.assign(n, -1);
    c->words.assign(experts_per_layer, uint64_t(kEmpty) << 32 | 0xffffffffu);
    c->dirty.assign(experts_per_layer, 0);
    if (out_errno) *out_errno = 0;
    return c;
}

static bool creation_arguments_ok(uint32_t slot_count, int policy, int *out_errno) {
    const char *what = nullptr;
    if (slot_count == 0) what = "slotCount must be positive";  // PreadExpertStreamer.swift:251
    else if (policy != SHRIKE_EVICT_AGING_LFU && policy != SHRIKE_EVICT_SLRU) what = "unknown eviction policy";
    if (!what) return true;
    set_error("%s", what);
    if (out_errno) *out_errno = EINVAL;
    return false;
}

shrike_slot_cache *shrike_slot_cache_create(uint32_t slot_count, uint32_t experts_per_layer, uint32_t first_cell,
                                            int policy, double slru_protected_share, int *out_errno) {
    if (!creation_arguments_ok(slot_count, policy, out_errno)) return nullptr;
    if (uint64_t(first_cell) + slot_count > 0xffffffffull) {
        set_error("cell range leaves 32 bits");
        if (out_errno) *out_errno = EINVAL;
        return nullptr;
    }
    shrike_cell_arena *arena = make_arena(first_cell + slot_count);
    if (!arena) {
        set_error("slot cache allocation failed");
        if (out_errno) *out_errno = ENOMEM;
        return nullptr;
    }
    return create_cache(arena, true, slot_count, experts_per_layer, first_cell, policy, slru_protected_share, out_errno);
}

shrike_slot_cache *shrike_slot_cache_create_in_arena(shrike_cell_arena *arena, uint32_t slot_count,
                                                     uint32_t experts_per_layer, uint32_t first_cell, int policy,
                                                     double slru_protected_share, int *out_errno) {
    if (!creation_arguments_ok(slot_count, policy, out_errno)) return nullptr;
    if (!arena || uint64_t(first_cell) + slot_count > arena->cell_count) {  // PreadExpertStreamer.swift:312-316
        set_error("the slots' cell range leaves the arena");
        if (out_errno) *out_errno = EINVAL;
        return nullptr;
    }
    return create_cache(arena, false, slot_count, experts_per_layer, first_cell, policy, slru_protected_share, out_errno);
}

void shrike_slot_cache_destroy(shrike_slot_cache *cache) { delete cache; }

int shrike_slot_cache_plan_with_landings(shrike_slot_cache *c, const int32_t *experts, uint32_t expert_count,
                                         int32_t layer, const int32_t *avoiding_slots, uint32_t avoiding_count,
                                         const uint8_t *protected_experts, uint32_t protected_count,
                                         const int32_t *gpu_missed_experts, uint32_t gpu_missed_count,
                                         const int32_t *leased_landings, uint32_t leased_count, int64_t misses_counted,
                                         shrike_expert_cache_plan *plan) {
    SHRIKE_REQUIRE(c && plan && (expert_count == 0 || experts), "expert cache plan: NULL argument");
    SHRIKE_REQUIRE(expert_count <= c->slot_count, "expert cache needs at least %u slots", expert_count);  // :419-420
    SHRIKE_REQUIRE(expert_count == 0 || (plan->experts && plan->assigned_slots && plan->assigned_generations && plan->misses),
                   "expert cache plan: an output array is NULL");
    SHRIKE_REQUIRE(avoiding_count == 0 || avoiding_slots, "expert cache plan: avoidingSlots is NULL");
    SHRIKE_REQUIRE(gpu_missed_count == 0 || gpu_missed_experts, "expert cache plan: gpuMissedExperts is NULL");
    SHRIKE_REQUIRE(leased_count == 0 || leased_landings, "expert cache plan: leasedLandings is NULL");
    SHRIKE_REQUIRE(leased_count == 0 || expert_count == 0 || (plan->adopted && plan->freed_experts && plan->freed_cells),
                   "expert cache plan: leased landings need the adopted and freed arrays");
    std::lock_guard<std::mutex> guard(c->lock);
    const int64_t clock = c->use_clock + 1;
    if (c->stats.plans > 0 && c->stats.plans % 1024 == 0)  // :433-438: aging
        for (auto &u : c->use_count) u >>= 1;
    c->reserve_loading();  // loading slots are neither hits nor victims, :441-443

    int32_t *assigned = plan->assigned_slots;
    uint32_t miss_count = 0;
    for (uint32_t i = 0; i < expert_count; ++i) {
        assigned[i] = -1;
        for (uint32_t s = 0; s < c->slot_count; ++s) {
            if (!c->reserved[s] && c->slot_state[s] == kResident && c->slot_expert[s] == experts[i]) {
                assigned[i] = int32_t(s);
                c->reserved[s] = 1;
                break;
            }
        }
        if (assigned[i] == -1) ++miss_count;
    }
    for (uint32_t i = 0; i < avoiding_count; ++i)
        if (avoiding_slots[i] >= 0 && uint32_t(avoiding_slots[i]) < c->slot_count) c->reserved[size_t(avoiding_slots[i])] = 1;

    if (miss_count > 0) {  // :461-467
        const bool protected_ok = protected_experts && c->select_victims(miss_count, protected_experts, protected_count);
        if (!protected_ok && !c->select_victims(miss_count, nullptr, 0)) {
            set_error("%u experts do not fit in %u cache slots (avoiding %u slots)", expert_count, c->slot_count, avoiding_count);
            return ENOSPC;
        }
    }

    c->use_clock = clock;
    for (uint32_t i = 0; i < expert_count; ++i)
        if (experts[i] >= 0 && size_t(experts[i]) < c->use_count.size()) ++c->use_count[size_t(experts[i])];
    for (uint32_t i = 0; i < expert_count; ++i)
        if (assigned[i] >= 0) c->slot_last_use[size_t(assigned[i])] = clock;
    if (c->slru)  // :476-481: an overflow slot's first hit ends its probation instead of promoting it
        for (uint32_t i = 0; i < expert_count; ++i) {
            if (assigned[i] < 0 || c->slot_protected[size_t(assigned[i])]) continue;
            if (c->overflow_probation[size_t(assigned[i])]) {
                c->overflow_probation[size_t(assigned[i])] = 0;
                continue;
            }
            c->promote(assigned[i], clock);
        }

    auto listed = [](const int32_t *list, uint32_t count, int32_t expert) {
        return list && std::find(list, list + count, expert) != list + count;
    };
    plan->miss_count = 0;
    plan->adopted_count = 0;
    plan->freed_count = 0;
    uint32_t victim_at = 0;
    for (uint32_t i = 0; i < expert_count; ++i) {
        if (assigned[i] != -1) continue;
        const int32_t slot = c->victims[victim_at++];
        if (c->slot_state[size_t(slot)] == kResident) ++c->stats.evictions;
        const int32_t previous = c->slot_expert[size_t(slot)];
        assigned[i] = slot;
        c->reserved[size_t(slot)] = 1;
        c->demote(slot);
        c->overflow_probation[size_t(slot)] = 0;
        const uint32_t cell = c->cell(slot);
        c->arena->bump(cell);
        if (previous >= 0) c->publish(previous, cell, kEmpty);
        // :499-515: a completed landing leased to this plan becomes the slot's cell without a
        // byte moving; the slot's old cell goes back to the ring
        const auto landing = listed(leased_landings, leased_count, experts[i]) ? c->landings.find(experts[i]) : c->landings.end();
        if (landing != c->landings.end() && landing->second.resident) {
            const uint32_t landed_cell = landing->second.cell;
            c->landings.erase(landing);
            plan->freed_experts[plan->freed_count] = experts[i];
            plan->freed_cells[plan->freed_count++] = cell;
            c->slot_cell[size_t(slot)] = landed_cell;
            c->slot_expert[size_t(slot)] = experts[i];
            c->slot_last_use[size_t(slot)] = clock;
            c->slot_state[size_t(slot)] = kResident;
            c->record_expert_load(experts[i]);
            if (listed(gpu_missed_experts, gpu_missed_count, experts[i])) plan->adopted[plan->adopted_count++] = i;
            continue;
        }
        c->slot_expert[size_t(slot)] = experts[i];
        c->slot_last_use[size_t(slot)] = clock;
        c->slot_state[size_t(slot)] = kLoading;
        c->publish(experts[i], cell, kLoading);
        plan->misses[plan->miss_count++] = i;
    }

    const uint64_t counted = misses_counted < 0 ? plan->miss_count : uint64_t(misses_counted);
    ++c->stats.plans;
    c->stats.requested_experts += expert_count;
    c->stats.hits += uint64_t(expert_count) - counted;
    c->stats.misses += counted;
    c->stats.peak_loading_slots = std::max(c->stats.peak_loading_slots, c->count_state(kLoading));

    plan->expert_count = expert_count;
    plan->layer = layer;
    plan->hits = expert_count - plan->miss_count;
    for (uint32_t i = 0; i < expert_count; ++i) {
        plan->experts[i] = experts[i];
        plan->assigned_generations[i] = c->generation_of(assigned[i]);
        if (plan->assigned_cells) plan->assigned_cells[i] = c->cell(assigned[i]);
    }
    return 0;
}

int shrike_slot_cache_plan(shrike_slot_cache *c, const int32_t *experts, uint32_t expert_count, int32_t layer,
                           const int32_t *avoiding_slots, uint32_t avoiding_count, const uint8_t *protected_experts,
                           uint32_t protected_count, int64_t misses_counted, shrike_expert_cache_plan *plan) {
    return shrike_slot_cache_plan_with_landings(c, experts, expert_count, layer, avoiding_slots, avoiding_count,
                                                protected_experts, protected_count, nullptr, 0, nullptr, 0, misses_counted,
                                                plan);
}

int shrike_slot_cache_complete(shrike_slot_cache *c, const shrike_expert_cache_plan *plan, uint64_t elapsed_nanos,
                               uint64_t fetch_nanos) {
    SHRIKE_REQUIRE(c && plan, "expert cache plan: NULL argument");
    std::lock_guard<std::mutex> guard(c->lock);
    for (uint32_t m = 0; m < plan->miss_count; ++m) {
        const uint32_t i = plan->misses[m];
        const int32_t slot = plan->assigned_slots[i];
        if (slot < 0 || uint32_t(slot) >= c->slot_count || c->generation_of(slot) != plan->assigned_generations[i]) {
            set_error("expert-cache cell generation changed during expert load");
            return EIO;
        }
    }
    for (uint32_t m = 0; m < plan->miss_count; ++m) {
        const uint32_t i = plan->misses[m];
        const int32_t slot = plan->assigned_slots[i];
        c->slot_state[size_t(slot)] = kResident;
        c->slot_expert[size_t(slot)] = plan->experts[i];
        c->slot_last_use[size_t(slot)] = c->use_clock;
        c->publish(plan->experts[i], c->cell(slot), kResident);
    }
    if (plan->miss_count == 0) return 0;
    // recordSuccessfulLoadsUnlocked, :1150-1179 (bytes are counted per read when reported)
    c->record_batch(plan->miss_count, elapsed_nanos, fetch_nanos);
    for (uint32_t m = 0; m < plan->miss_count; ++m) c->record_expert_load(plan->experts[plan->misses[m]]);
    return 0;
}

void shrike_slot_cache_abandon(shrike_slot_cache *c, const shrike_expert_cache_plan *plan) {
    if (!c || !plan) return;
    std::lock_guard<std::mutex> guard(c->lock);
    for (uint32_t m = 0; m < plan->miss_count; ++m) {
        const uint32_t i = plan->misses[m];
        const int32_t slot = plan->assigned_slots[i];
        if (slot < 0 || uint32_t(slot) >= c->slot_count || c->generation_of(slot) != plan->assigned_generations[i] ||
            c->slot_state[size_t(slot)] != kLoading)
            continue;
        c->slot_state[size_t(slot)] = kEmpty;
        c->slot_expert[size_t(slot)] = -1;
        c->publish(plan->experts[i], c->cell(slot), kEmpty);
    }
}

int shrike_slot_cache_pin(shrike_slot_cache *c, const shrike_expert_cache_plan *plan) {
    SHRIKE_REQUIRE(c && plan, "expert cache plan: NULL argument");
    std::lock_guard<std::mutex> guard(c->lock);
    for (uint32_t i = 0; i < plan->expert_count; ++i) {
        const int32_t slot = plan->assigned_slots[i];
        if (slot < 0 || uint32_t(slot) >= c->slot_count || c->generation_of(slot) != plan->assigned_generations[i] ||
            c->slot_expert[size_t(slot)] != plan->experts[i] || c->slot_state[size_t(slot)] == kEmpty) {
            set_error("expert-cache plan became stale before GPU pin");
            return EIO;
        }
    }
    for (uint32_t i = 0; i < plan->expert_count; ++i) ++c->slot_pins[size_t(plan->assigned_slots[i])];
    return 0;
}

void shrike_slot_cache_unpin(shrike_slot_cache *c, const int32_t *slots, const uint64_t *generations, uint32_t count) {
    if (!c || !slots || !generations) return;
    std::lock_guard<std::mutex> guard(c->lock);
    for (uint32_t i = 0; i < count; ++i) {
        const int32_t slot = slots[i];
        if (slot < 0 || uint32_t(slot) >= c->slot_count || c->generation_of(slot) != generations[i]) continue;
        if (c->slot_pins[size_t(slot)] > 0) --c->slot_pins[size_t(slot)];
    }
}

int64_t shrike_slot_cache_slot_cell(shrike_slot_cache *c, uint32_t slot) {
    if (!c || slot >= c->slot_count) return -1;
    std::lock_guard<std::mutex> guard(c->lock);
    return c->cell(int32_t(slot));
}

int shrike_slot_cache_owns_cell(shrike_slot_cache *c, uint32_t cell) {
    if (!c) return 0;
    std::lock_guard<std::mutex> guard(c->lock);
    return c->slot_of_cell(cell) >= 0;
}

// claimLanding's body, under the lock
static bool claim_landing(shrike_slot_cache *c, int32_t expert, int64_t cell) {
    if (expert < 0 || uint32_t(expert) >= c->experts_per_layer || cell < 0 || cell >= int64_t(c->arena->cell_count)) return false;
    if (c->landings.count(expert) || c->holds(expert)) return false;
    for (const auto &entry : c->landings)
        if (entry.second.cell == uint32_t(cell)) return false;
    c->landings[expert] = Landing{uint32_t(cell), false, c->arena->bump(uint32_t(cell))};
    c->publish(expert, uint32_t(cell), kLoading);
    return true;
}

static void drop_landing(shrike_slot_cache *c, int32_t expert, int64_t cell) {
    const auto landing = c->landings.find(expert);
    if (landing == c->landings.end() || int64_t(landing->second.cell) != cell) return;
    c->landings.erase(landing);
    if (!c->holds(expert)) c->publish(expert, uint32_t(cell), kEmpty);
}

int shrike_slot_cache_claim_landing(shrike_slot_cache *c, int32_t expert, int64_t cell) {
    if (!c) return 0;
    std::lock_guard<std::mutex> guard(c->lock);
    return claim_landing(c, expert, cell);
}

int shrike_slot_cache_complete_landing(shrike_slot_cache *c, int32_t expert, int64_t cell) {
    if (!c) return 0;
    std::lock_guard<std::mutex> guard(c->lock);
    const auto landing = c->landings.find(expert);
    if (landing == c->landings.end() || int64_t(landing->second.cell) != cell || landing->second.resident ||
        c->arena->generation(uint32_t(cell)) != landing->second.generation)
        return 0;
    if (c->holds(expert)) {  // the pool overtook the landing with its own read: the pool's entry stands
        c->landings.erase(landing);
        return 0;
    }
    landing->second.resident = true;
    c->publish(expert, uint32_t(cell), kResident);
    return 1;
}

void shrike_slot_cache_drop_landing(shrike_slot_cache *c, int32_t expert, int64_t cell) {
    if (!c) return;
    std::lock_guard<std::mutex> guard(c->lock);
    drop_landing(c, expert, cell);
}

void shrike_slot_cache_fail_landing(shrike_slot_cache *c, int32_t expert, int64_t cell) {
    shrike_slot_cache_drop_landing(c, expert, cell);
}

int shrike_slot_cache_claim_prefetch(shrike_slot_cache *c, const int32_t *experts, const int64_t *cells, uint32_t count,
                                     uint32_t *refused_index) {
    SHRIKE_REQUIRE(c && (count == 0 || (experts && cells)), "prefetch: NULL argument");
    std::lock_guard<std::mutex> guard(c->lock);
    for (uint32_t i = 0; i < count; ++i)
        SHRIKE_REQUIRE(experts[i] >= 0 && uint32_t(experts[i]) < c->experts_per_layer, "invalid prefetched expert");
    for (uint32_t i = 0; i < count; ++i)
        SHRIKE_REQUIRE(cells[i] < 0 || cells[i] > 0xffffffffll || c->slot_of_cell(uint32_t(cells[i])) < 0,
                       "a prefetch landing was offered cell %lld, which the pool owns", (long long)cells[i]);
    for (uint32_t i = 0; i < count; ++i) {
        if (claim_landing(c, experts[i], cells[i])) continue;
        for (uint32_t j = 0; j < i; ++j) drop_landing(c, experts[j], cells[j]);
        if (refused_index) *refused_index = i;
        set_error("prefetch claim refused: expert %d, cell %lld", experts[i], (long long)cells[i]);
        return SHRIKE_PREFETCH_CLAIM_REFUSED;
    }
    return 0;
}

int64_t shrike_slot_cache_reserve_overflow_slot(shrike_slot_cache *c, int32_t expert, const int32_t *protecting,
                                                uint32_t protecting_count) {
    if (!c || expert < 0 || uint32_t(expert) >= c->experts_per_layer || (protecting_count && !protecting)) return -1;
    std::lock_guard<std::mutex> guard(c->lock);
    if (c->holds(expert)) return -1;
    c->reserve_loading();
    for (uint32_t s = 0; s < c->slot_count; ++s)
        if (c->slot_state[s] == kResident &&
            std::find(protecting, protecting + protecting_count, c->slot_expert[s]) != protecting + protecting_count)
            c->reserved[s] = 1;
    if (!c->select_victims(1, nullptr, 0)) return -1;
    const int32_t slot = c->victims[0];
    c->overflow_probation[size_t(slot)] = 1;
    if (c->slot_state[size_t(slot)] == kResident) ++c->stats.evictions;
    const int32_t previous = c->slot_expert[size_t(slot)];
    c->demote(slot);
    const uint32_t cell = c->cell(slot);
    c->arena->bump(cell);
    if (previous >= 0) c->publish(previous, cell, kEmpty);
    c->slot_expert[size_t(slot)] = expert;
    c->slot_last_use[size_t(slot)] = c->use_clock;
    c->slot_state[size_t(slot)] = kLoading;
    c->publish(expert, cell, kLoading);
    return cell;
}

void shrike_slot_cache_mark_overflow_resident(shrike_slot_cache *c, int32_t expert, int64_t cell) {
    if (!c || cell < 0 || cell > 0xffffffffll) return;
    std::lock_guard<std::mutex> guard(c->lock);
    const int32_t slot = c->slot_of_cell(uint32_t(cell));
    if (slot < 0 || c->slot_state[size_t(slot)] != kLoading || c->slot_expert[size_t(slot)] != expert) return;
    c->slot_state[size_t(slot)] = kResident;
    c->slot_last_use[size_t(slot)] = c->use_clock;
    c->publish(expert, uint32_t(cell), kResident);
}

void shrike_slot_cache_abandon_overflow_slot(shrike_slot_cache *c, int32_t expert, int64_t cell) {
    if (!c || cell < 0 || cell > 0xffffffffll) return;
    std::lock_guard<std::mutex> guard(c->lock);
    const int32_t slot = c->slot_of_cell(uint32_t(cell));
    if (slot < 0 || c->slot_state[size_t(slot)] != kLoading || c->slot_expert[size_t(slot)] != expert) return;
    c->slot_state[size_t(slot)] = kEmpty;
    c->slot_expert[size_t(slot)] = -1;
    c->overflow_probation[size_t(slot)] = 0;
    c->publish(expert, uint32_t(cell), kEmpty);
}

int shrike_slot_cache_finish_agreed_reads(shrike_slot_cache *c, const int32_t *experts, const int64_t *cells, uint32_t count,
                                          int succeeded, uint64_t elapsed_nanos, uint64_t fetch_nanos) {
    SHRIKE_REQUIRE(c && (count == 0 || (experts && cells)), "agreed reads: NULL argument");
    // which cells were the pool's is settled before any of them changes state, as in beginAgreedReads
    std::vector<uint8_t> pool_cell(count, 0);
    {
        std::lock_guard<std::mutex> guard(c->lock);
        for (uint32_t i = 0; i < count; ++i) {
            SHRIKE_REQUIRE(experts[i] >= 0 && uint32_t(experts[i]) < c->experts_per_layer && cells[i] >= 0 &&
                               cells[i] < int64_t(c->arena->cell_count),
                           "invalid agreed read");
            pool_cell[i] = c->slot_of_cell(uint32_t(cells[i])) >= 0;
        }
    }
    for (uint32_t i = 0; i < count; ++i) {
        if (succeeded) {
            if (pool_cell[i]) shrike_slot_cache_mark_overflow_resident(c, experts[i], cells[i]);
            else shrike_slot_cache_complete_landing(c, experts[i], cells[i]);
        } else {
            if (pool_cell[i]) shrike_slot_cache_abandon_overflow_slot(c, experts[i], cells[i]);
            else shrike_slot_cache_fail_landing(c, experts[i], cells[i]);
        }
    }
    if (!succeeded || count == 0) return 0;
    std::lock_guard<std::mutex> guard(c->lock);  // recordAgreedLoads, :994-1002
    c->record_batch(count, elapsed_nanos, fetch_nanos);
    for (uint32_t i = 0; i < count; ++i)
        if (pool_cell[i]) c->record_expert_load(experts[i]);
    return 0;
}

void shrike_slot_cache_statistics(shrike_slot_cache *c, uint64_t expert_stride_bytes, shrike_streaming_statistics *out) {
    if (!c || !out) return;
    std::lock_guard<std::mutex> guard(c->lock);
    *out = c->stats;
    out->bytes_read = c->stats.read_operations * expert_stride_bytes;
    out->resident_slots = c->count_state(kResident);
    out->loading_slots = c->count_state(kLoading);
    out->pinned_slots = uint32_t(std::count_if(c->slot_pins.begin(), c->slot_pins.end(), [](int64_t p) { return p > 0; }));
}

size_t shrike_slot_cache_resident_experts(shrike_slot_cache *c, int32_t *out, size_t capacity) {
    if (!c) return 0;
    std::lock_guard<std::mutex> guard(c->lock);
    std::vector<int32_t> ids;
    for (uint32_t s = 0; s < c->slot_count; ++s)
        if (c->slot_state[s] == kResident && c->slot_expert[s] >= 0) ids.push_back(c->slot_expert[s]);
    std::sort(ids.begin(), ids.end());
    for (size_t i = 0; i < ids.size() && i < capacity && out; ++i) out[i] = ids[i];
    return ids.size();
}

uint64_t shrike_slot_cache_entry(shrike_slot_cache *c, uint32_t expert) {
    if (!c || expert >= c->experts_per_layer) return uint64_t(kEmpty) << 32 | 0xffffffffu;
    std::lock_guard<std::mutex> guard(c->lock);
    return c->words[expert];
}

size_t shrike_slot_cache_drain_publications(shrike_slot_cache *c, uint32_t *experts, uint64_t *words, size_t capacity) {
    if (!c || !experts || !words) return 0;
    std::lock_guard<std::mutex> guard(c->lock);
    const size_t n = std::min(capacity, c->dirty_order.size());
    for (size_t i = 0; i < n; ++i) {
        const uint32_t e = c->dirty_order[i];
        experts[i] = e;
        words[i] = c->words[e];
        c->dirty[e] = 0;
    }
    c->dirty_order.erase(c->dirty_order.begin(), c->dirty_order.begin() + ptrdiff_t(n));
    return n;
}

}  // extern "C"
