// The routed-tile loop of a prefill chunk whose experts stream through a slot pool: the
// scheduler's decisions (PrefillRoutedTileScheduler.swift), the loop that drives plans, begun
// fetches, encodes, batches and drains in the reference's order (PrefillRoutedTileSequencer.swift),
// the chunk's victim protection (RealForwardRunner.swift:63-93) and the slot-lifetime guard
// (PrefillGroupedRoutedMoE.swift:388-424). Pure host logic: every effect is the driver's.
#include <algorithm>
#include <map>
#include <set>
#include <vector>

#include "../../include/shrike_host.h"
#include "host_common.h"

using shrike::set_error;

namespace {

int clampi(int v, int lo, int hi) { return std::max(lo, std::min(hi, v)); }
int in_flight_batches(const shrike_tile_scheduler_config &c) { return c.max_pending_depth + 1; }
int max_in_flight_tiles(const shrike_tile_scheduler_config &c) {
    return in_flight_batches(c) * c.tiles_per_command_buffer + c.fetch_lookahead;
}

// PrefillRoutedTileSequencer.issue, PrefillRoutedTileSequencer.swift:87-104
int issue(const shrike_tile_scheduler_config &config, const shrike_tile_driver &d, int tile, bool plan_available) {
    const int depth = d.pending_depth(d.context);
    const int decision = shrike_tile_scheduler_decide(&config, depth > 0, depth, d.pending_assigned_slot_count(d.context), plan_available);
    if (decision >= SHRIKE_TILE_DRAIN_NO_ASSIGNED_SLOTS) {
        if (plan_available)
            if (int rc = d.abandon_plan(d.context, tile)) return rc;
        if (int rc = d.drain_oldest_batch(d.context)) return rc;
    }
    return d.begin(d.context, tile);
}

// PrefillRoutedTileSequencer.sequence, PrefillRoutedTileSequencer.swift:39-85
int sequence(const shrike_tile_scheduler_config &config, int tile_count, const shrike_tile_driver &d) {
    int carried = -1;
    for (int tile = 0; tile < tile_count; ++tile) {
        const bool is_last = tile == tile_count - 1;
        const bool carried_fetch = carried == tile;
        carried = -1;
        int plan_available = 1;
        if (!carried_fetch)
            if (int rc = d.plan(d.context, tile, -1, &plan_available)) return rc;
        shrike_tile_batch_action action;
        shrike_tile_scheduler_batch_action(&config, d.open_batch_tiles(d.context), d.open_batch_slot_count(d.context), plan_available,
                                           is_last, &action);
        if (action.commit_before_append) d.commit_open_batch(d.context);
        if (!carried_fetch)
            if (int rc = issue(config, d, tile, plan_available != 0)) return rc;
        if (shrike_tile_scheduler_plans_lookahead(&config, tile, tile_count)) {
            const int successor = tile + 1;
            int successor_available = 0;
            if (int rc = d.plan(d.context, successor, tile, &successor_available)) return rc;
            if (shrike_tile_scheduler_should_begin_lookahead(&config, tile, tile_count, successor_available)) {
                if (int rc = d.begin(d.context, successor)) return rc;
                carried = successor;
            }
        }
        if (int rc = d.encode(d.context, tile)) return rc;
        if (action.commit_after_append != SHRIKE_TILE_BATCH_OPEN) d.commit_open_batch(d.context);
        // a still-open batch holds the tile just encoded and counts against the depth with the committed ones
        while (d.pending_depth(d.context) + (d.open_batch_tiles(d.context) > 0 ? 1 : 0) > config.max_pending_depth)
            if (int rc = d.drain_oldest_batch(d.context)) return rc;
    }
    d.commit_open_batch(d.context);
    while (d.pending_depth(d.context) > 0)
        if (int rc = d.drain_oldest_batch(d.context)) return rc;
    return 0;
}

}  // namespace

struct shrike_tile_lifetime {
    std::map<int, std::set<int>> in_flight;  // tile -> its slots
};

extern "C" {

void shrike_tile_scheduler_config_make(int max_pending_depth, int tile_experts, int tiles_per_command_buffer, int fetch_lookahead,
                                       shrike_tile_scheduler_config *out) {
    // PrefillRoutedTileSchedulerConfig.init, PrefillRoutedTileScheduler.swift:52-58
    out->max_pending_depth = std::max(1, max_pending_depth);
    out->tile_experts = clampi(tile_experts, 1, 16);
    out->tiles_per_command_buffer = clampi(tiles_per_command_buffer, 1, 16);
    out->fetch_lookahead = clampi(fetch_lookahead, 0, 1);
}

int shrike_tile_scheduler_fits_slot_budget(const shrike_tile_scheduler_config *c, int slot_count, int reserved_hits) {
    if (!(slot_count > 0 && reserved_hits >= 0)) return 0;  // :63-66
    return max_in_flight_tiles(*c) * c->tile_experts + reserved_hits <= slot_count;
}

int shrike_tile_scheduler_fitting(const shrike_tile_scheduler_config *c, int slot_count, int reserved_hits,
                                  shrike_tile_scheduler_config *out) {
    // :71-91: the batch width narrows first, then the tile
    if (!(slot_count > reserved_hits && reserved_hits >= 0)) return 0;
    const int available = slot_count - reserved_hits;
    shrike_tile_scheduler_config narrowed;
    shrike_tile_scheduler_config_make(
        c->max_pending_depth, c->tile_experts,
        std::max(1, std::min(c->tiles_per_command_buffer,
                             (available - c->fetch_lookahead * c->tile_experts) / (in_flight_batches(*c) * c->tile_experts))),
        c->fetch_lookahead, &narrowed);
    if (shrike_tile_scheduler_fits_slot_budget(&narrowed, slot_count, reserved_hits)) {
        *out = narrowed;
        return 1;
    }
    const int per_tile = available / (in_flight_batches(*c) + c->fetch_lookahead);
    if (per_tile <= 0) return 0;
    shrike_tile_scheduler_config_make(c->max_pending_depth, std::min(c->tile_experts, per_tile), 1, c->fetch_lookahead, out);
    return 1;
}

int shrike_tile_scheduler_decide(const shrike_tile_scheduler_config *c, int has_pending_tile, int pending_depth,
                                 size_t pending_assigned_slot_count, int avoiding_slot_plan_available) {
    // PrefillRoutedTileSchedulerInput.init (:36-44) and decide (:104-122)
    const int depth = std::max(0, pending_depth < 0 ? (has_pending_tile ? 1 : 0) : pending_depth);
    if (!has_pending_tile) return SHRIKE_TILE_ISSUE_WITHOUT_PENDING;
    if (depth > c->max_pending_depth) return SHRIKE_TILE_DRAIN_MAX_DEPTH;
    if (pending_assigned_slot_count == 0) return SHRIKE_TILE_DRAIN_NO_ASSIGNED_SLOTS;
    if (!avoiding_slot_plan_available) return SHRIKE_TILE_DRAIN_PLAN_UNAVAILABLE;
    return SHRIKE_TILE_PREFETCH_NEXT;
}

int shrike_tile_scheduler_plans_lookahead(const shrike_tile_scheduler_config *c, int index, int tile_count) {
    return c->fetch_lookahead > 0 && index + 1 < tile_count;  // :126-128
}

int shrike_tile_scheduler_should_begin_lookahead(const shrike_tile_scheduler_config *c, int index, int tile_count,
                                                 int avoiding_slot_plan_available) {
    return shrike_tile_scheduler_plans_lookahead(c, index, tile_count) && avoiding_slot_plan_available;  // :133-137
}

void shrike_tile_scheduler_batch_action(const shrike_tile_scheduler_config *c, int open_batch_tiles, size_t open_batch_slot_count,
                                        int next_tile_plan_available, int is_last_tile, shrike_tile_batch_action *out) {
    // :139-155
    const bool before = open_batch_slot_count != 0 && !next_tile_plan_available;
    const int tiles_after = (before ? 0 : std::max(0, open_batch_tiles)) + 1;
    out->commit_before_append = before ? 1 : 0;
    out->commit_after_append = tiles_after >= c->tiles_per_command_buffer ? SHRIKE_TILE_BATCH_FULL
                               : is_last_tile                             ? SHRIKE_TILE_BATCH_LAST_TILE
                                                                          : SHRIKE_TILE_BATCH_OPEN;
}

int shrike_tile_sequencer_run(const shrike_tile_scheduler_config *config, int tile_count, const shrike_tile_driver *driver) {
    SHRIKE_REQUIRE(config && driver, "tile sequencer: config or driver is NULL");
    SHRIKE_REQUIRE(driver->open_batch_tiles && driver->open_batch_slot_count && driver->pending_depth
                       && driver->pending_assigned_slot_count && driver->plan && driver->begin && driver->abandon_plan && driver->encode
                       && driver->commit_open_batch && driver->drain_oldest_batch && driver->abandon_begun_fetches,
                   "tile sequencer: the driver leaves a callback unset");
    const int rc = sequence(*config, tile_count, *driver);
    if (rc != 0) driver->abandon_begun_fetches(driver->context);  // PrefillRoutedTileSequencer.swift:30-37
    return rc;
}

void shrike_chunk_protection_init(const int32_t *routed_experts, size_t count, uint8_t *remaining, size_t experts_per_layer) {
    std::fill(remaining, remaining + experts_per_layer, uint8_t(0));
    for (size_t i = 0; i < count; ++i)
        if (routed_experts[i] >= 0 && size_t(routed_experts[i]) < experts_per_layer) remaining[routed_experts[i]] = 1;
}

void shrike_chunk_protection_planning(const int32_t *tile_experts, size_t count, uint8_t *remaining, size_t experts_per_layer) {
    for (size_t i = 0; i < count; ++i)
        if (tile_experts[i] >= 0 && size_t(tile_experts[i]) < experts_per_layer) remaining[tile_experts[i]] = 0;
}

shrike_tile_lifetime *shrike_tile_lifetime_create(void) { return new shrike_tile_lifetime(); }
void shrike_tile_lifetime_destroy(shrike_tile_lifetime *lifetime) { delete lifetime; }

int shrike_tile_lifetime_begin(shrike_tile_lifetime *lifetime, int tile_index, const int32_t *planned_slots, size_t count,
                               int *conflicting_tile) {
    if (conflicting_tile) *conflicting_tile = -1;
    if (!lifetime || (count && !planned_slots)) return SHRIKE_TILE_LIFETIME_INVALID;
    std::set<int> slots;
    for (size_t i = 0; i < count; ++i)
        if (!slots.insert(planned_slots[i]).second) {
            set_error("tile %d plans slot %d twice", tile_index, planned_slots[i]);
            return SHRIKE_TILE_LIFETIME_DUPLICATE_SLOTS;
        }
    for (const auto &other : lifetime->in_flight)
        for (int slot : slots)
            if (other.second.count(slot)) {
                if (conflicting_tile) *conflicting_tile = other.first;
                set_error("tile %d reuses slot %d before tile %d has completed", tile_index, slot, other.first);
                return SHRIKE_TILE_LIFETIME_SLOT_REUSE;
            }
    lifetime->in_flight[tile_index] = std::move(slots);
    return 0;
}

int shrike_tile_lifetime_complete(shrike_tile_lifetime *lifetime, int tile_index) {
    if (!lifetime) return SHRIKE_TILE_LIFETIME_INVALID;
    if (lifetime->in_flight.erase(tile_index) == 0) {
        set_error("tile %d completes without being in flight", tile_index);
        return SHRIKE_TILE_LIFETIME_NOT_IN_FLIGHT;
    }
    return 0;
}

}  // extern "C"
