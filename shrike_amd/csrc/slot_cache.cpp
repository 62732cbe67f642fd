// The slot cache's bookkeeping: which expert sits in which slot of the HBM pool, which
// slot a miss may take, and the residency words the kernels classify against
// (PreadExpertStreamer.swift:405-543, :676-767, :1085-1148). No device calls: the owner
// mirrors the drained publications into the pool's device table.
#include <algorithm>
#include <cmath>
#include <mutex>
#include <vector>

#include "../../include/shrike_host.h"
#include "host_common.h"

using shrike::set_error;

namespace {
enum : uint8_t { kEmpty = 0, kLoading = 1, kResident = 2 };
}

struct shrike_slot_cache {
    uint32_t slot_count, experts_per_layer, first_cell;
    bool slru;
    int64_t protected_capacity;
    std::mutex lock;
    std::vector<int32_t> slot_expert;
    std::vector<int64_t> slot_last_use;
    std::vector<uint8_t> slot_state, slot_protected, reserved;
    std::vector<int64_t> slot_pins;
    std::vector<int64_t> use_count, load_count;
    std::vector<uint64_t> generation;
    std::vector<int32_t> victims;
    std::vector<uint64_t> words;
    std::vector<uint8_t> dirty;
    std::vector<uint32_t> dirty_order;
    uint64_t generation_clock = 0;
    int64_t use_clock = 0;
    int64_t protected_count = 0;
    shrike_streaming_statistics stats{};

    uint32_t cell(int32_t slot) const { return first_cell + uint32_t(slot); }

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

shrike_slot_cache *shrike_slot_cache_create(uint32_t slot_count, uint32_t experts_per_layer, uint32_t first_cell,
                                            int policy, double slru_protected_share, int *out_errno) {
    auto fail = [&](int code, const char *what) -> shrike_slot_cache * {
        set_error("%s", what);
        if (out_errno) *out_errno = code;
        return nullptr;
    };
    if (slot_count == 0) return fail(EINVAL, "slotCount must be positive");  // PreadExpertStreamer.swift:249
    if (policy != SHRIKE_EVICT_AGING_LFU && policy != SHRIKE_EVICT_SLRU) return fail(EINVAL, "unknown eviction policy");
    if (uint64_t(first_cell) + slot_count > 0xffffffffull) return fail(EINVAL, "cell range leaves 32 bits");
    auto *c = new (std::nothrow) shrike_slot_cache();
    if (!c) return fail(ENOMEM, "slot cache allocation failed");
    c->slot_count = slot_count;
    c->experts_per_layer = experts_per_layer;
    c->first_cell = first_cell;
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
    c->generation.assign(n, 0);
    c->victims.assign(n, -1);
    c->words.assign(experts_per_layer, uint64_t(kEmpty) << 32 | 0xffffffffu);
    c->dirty.assign(experts_per_layer, 0);
    if (out_errno) *out_errno = 0;
    return c;
}

void shrike_slot_cache_destroy(shrike_slot_cache *cache) { delete cache; }

int shrike_slot_cache_plan(shrike_slot_cache *c, const int32_t *experts, uint32_t expert_count, int32_t layer,
                           const int32_t *avoiding_slots, uint32_t avoiding_count, const uint8_t *protected_experts,
                           uint32_t protected_count, int64_t misses_counted, shrike_expert_cache_plan *plan) {
    SHRIKE_REQUIRE(c && plan && (expert_count == 0 || experts), "expert cache plan: NULL argument");
    SHRIKE_REQUIRE(expert_count <= c->slot_count, "expert cache needs at least %u slots", expert_count);  // :419-420
    SHRIKE_REQUIRE(expert_count == 0 || (plan->experts && plan->assigned_slots && plan->assigned_generations && plan->misses),
                   "expert cache plan: an output array is NULL");
    SHRIKE_REQUIRE(avoiding_count == 0 || avoiding_slots, "expert cache plan: avoidingSlots is NULL");
    std::lock_guard<std::mutex> guard(c->lock);
    std::fill(c->reserved.begin(), c->reserved.end(), 0);
    const int64_t clock = c->use_clock + 1;
    if (c->stats.plans > 0 && c->stats.plans % 1024 == 0)  // :433-438: aging
        for (auto &u : c->use_count) u >>= 1;
    for (uint32_t s = 0; s < c->slot_count; ++s)
        if (c->slot_state[s] == kLoading) c->reserved[s] = 1;

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
    if (c->slru)
        for (uint32_t i = 0; i < expert_count; ++i)
            if (assigned[i] >= 0 && !c->slot_protected[size_t(assigned[i])]) c->promote(assigned[i], clock);

    plan->miss_count = 0;
    uint32_t victim_at = 0;
    for (uint32_t i = 0; i < expert_count; ++i) {
        if (assigned[i] != -1) continue;
        const int32_t slot = c->victims[victim_at++];
        if (c->slot_state[size_t(slot)] == kResident) ++c->stats.evictions;
        const int32_t previous = c->slot_expert[size_t(slot)];
        assigned[i] = slot;
        c->reserved[size_t(slot)] = 1;
        if (c->slot_protected[size_t(slot)]) {
            c->slot_protected[size_t(slot)] = 0;
            --c->protected_count;
        }
        c->generation[size_t(slot)] = ++c->generation_clock;  // ExpertCellArena.swift:99-104
        if (previous >= 0) c->publish(previous, c->cell(slot), kEmpty);
        c->slot_expert[size_t(slot)] = experts[i];
        c->slot_last_use[size_t(slot)] = clock;
        c->slot_state[size_t(slot)] = kLoading;
        c->publish(experts[i], c->cell(slot), kLoading);
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
        plan->assigned_generations[i] = c->generation[size_t(assigned[i])];
    }
    return 0;
}

int shrike_slot_cache_complete(shrike_slot_cache *c, const shrike_expert_cache_plan *plan, uint64_t elapsed_nanos,
                               uint64_t fetch_nanos) {
    SHRIKE_REQUIRE(c && plan, "expert cache plan: NULL argument");
    std::lock_guard<std::mutex> guard(c->lock);
    for (uint32_t m = 0; m < plan->miss_count; ++m) {
        const uint32_t i = plan->misses[m];
        const int32_t slot = plan->assigned_slots[i];
        if (slot < 0 || uint32_t(slot) >= c->slot_count || c->generation[size_t(slot)] != plan->assigned_generations[i]) {
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
    c->stats.read_operations += plan->miss_count;
    ++c->stats.load_batches;
    c->stats.total_load_nanos += elapsed_nanos;
    c->stats.fetch_nanos += fetch_nanos;
    c->stats.maximum_load_nanos = std::max(c->stats.maximum_load_nanos, elapsed_nanos);
    uint64_t bound = 125000;  // latencyBucketIndex, :1181-1188
    int bucket = 16;
    for (int index = 0; index < 16; ++index) {
        if (elapsed_nanos <= bound) {
            bucket = index;
            break;
        }
        bound *= 2;
    }
    ++c->stats.latency_histogram[bucket];
    for (uint32_t m = 0; m < plan->miss_count; ++m) {
        const int32_t e = plan->experts[plan->misses[m]];
        if (e < 0 || size_t(e) >= c->load_count.size()) continue;
        if (c->load_count[size_t(e)] > 0) ++c->stats.reloads;
        ++c->load_count[size_t(e)];
    }
    return 0;
}

void shrike_slot_cache_abandon(shrike_slot_cache *c, const shrike_expert_cache_plan *plan) {
    if (!c || !plan) return;
    std::lock_guard<std::mutex> guard(c->lock);
    for (uint32_t m = 0; m < plan->miss_count; ++m) {
        const uint32_t i = plan->misses[m];
        const int32_t slot = plan->assigned_slots[i];
        if (slot < 0 || uint32_t(slot) >= c->slot_count || c->generation[size_t(slot)] != plan->assigned_generations[i] ||
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
        if (slot < 0 || uint32_t(slot) >= c->slot_count || c->generation[size_t(slot)] != plan->assigned_generations[i] ||
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
        if (slot < 0 || uint32_t(slot) >= c->slot_count || c->generation[size_t(slot)] != generations[i]) continue;
        if (c->slot_pins[size_t(slot)] > 0) --c->slot_pins[size_t(slot)];
    }
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
