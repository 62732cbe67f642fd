// Load operations and the predictive prefetch ring of the expert streamer, as host logic with no
// device calls (sources/Shrike/Infrastructure/Streaming/ExpertLoadOperation.swift,
// sources/Shrike/Runtime/Inference/ExpertPrefetchRing.swift). The ring owns a few cells of the expert
// pool; predicted experts are read into them ahead of their layer, a plan that wants a landing swaps
// it into the layer's pool (the ring takes the freed cell), one nobody wants is dropped from the
// layer's residency table before its cell is read into again.
#include <time.h>

#include <atomic>
#include <cerrno>
#include <condition_variable>
#include <cstdint>
#include <mutex>
#include <new>
#include <thread>
#include <vector>

#include "../../include/shrike_host.h"

namespace {

uint64_t now_nanos() {
    timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return uint64_t(ts.tv_sec) * 1000000000ull + uint64_t(ts.tv_nsec);
}

}  // namespace

// ExpertLoadOperation.swift:15-153. The terminal transition happens once; waiters block on the
// condition. Shared by the submitter, the storage thread and the ring: reference counted.
struct shrike_load_operation {
    std::mutex lock;
    std::condition_variable changed;
    int state = SHRIKE_LOAD_SUBMITTED;
    int failure = 0;
    uint64_t submitted = 0, started = 0, completed = 0;
    std::atomic<int> references{1};
};

namespace {

int state_of(shrike_load_operation *op) {
    std::lock_guard<std::mutex> held(op->lock);
    return op->state;
}

bool terminal(int state) { return state == SHRIKE_LOAD_COMPLETED || state == SHRIKE_LOAD_FAILED; }

struct Slot {  // ExpertPrefetchRing.swift:51-72
    int cell = 0;
    int layer = -1, expert = -1;
    shrike_load_operation *operation = nullptr;  // retained
    bool leased = false, demand = false;
};

}  // namespace

struct shrike_prefetch_ring {
    std::mutex lock;
    std::vector<Slot> slots;
    shrike_prefetch_drop drop = nullptr;
    void *drop_context = nullptr;
    shrike_prefetch_statistics stats = {};

    void attach(Slot &slot, shrike_load_operation *op) {
        if (op) shrike_load_operation_retain(op);
        if (slot.operation) shrike_load_operation_release(slot.operation);
        slot.operation = op;
    }
    void clear(Slot &slot) {
        slot.layer = -1;
        slot.expert = -1;
        attach(slot, nullptr);
    }
    // :60-71: a claimed slot whose operation is not attached yet is in flight too
    bool in_flight(const Slot &slot) const {
        if (slot.expert < 0) return false;
        return !slot.operation || !terminal(state_of(slot.operation));
    }
    int in_flight_count() const {
        int n = 0;
        for (const Slot &slot : slots) n += in_flight(slot) ? 1 : 0;
        return n;
    }
    int leased_count() const {
        int n = 0;
        for (const Slot &slot : slots) n += slot.leased ? 1 : 0;
        return n;
    }
    // :333-351
    void reclaim_terminal(int keeping_layer) {
        for (Slot &slot : slots) {
            if (slot.leased || slot.layer == keeping_layer || !slot.operation) continue;
            const int state = state_of(slot.operation);
            if (state == SHRIKE_LOAD_COMPLETED) {
                if (drop) drop(drop_context, slot.layer, slot.expert, slot.cell);
                ++stats.reclaimed;
                clear(slot);
            } else if (state == SHRIKE_LOAD_FAILED) {
                ++stats.failed;
                clear(slot);
            }
        }
    }
};

namespace {

bool contains(const int *values, size_t count, int value) {
    for (size_t i = 0; i < count; ++i)
        if (values[i] == value) return true;
    return false;
}

// :216-228: the slot's operation (retained for the caller), waiting briefly for an issue in progress
// on another thread to attach it. Called and returns with the ring locked.
shrike_load_operation *attached_operation(shrike_prefetch_ring *ring, std::unique_lock<std::mutex> &held, size_t index) {
    Slot &slot = ring->slots[index];
    const int layer = slot.layer, expert = slot.expert;
    const uint64_t deadline = now_nanos() + SHRIKE_PREFETCH_ATTACH_SPIN_NANOS;
    while (!slot.operation && now_nanos() < deadline) {
        held.unlock();
        std::this_thread::sleep_for(std::chrono::microseconds(50));
        held.lock();
        if (slot.layer != layer || slot.expert != expert) return nullptr;
    }
    if (slot.operation) shrike_load_operation_retain(slot.operation);
    return slot.operation;
}

}  // namespace

extern "C" {

uint64_t shrike_monotonic_nanos(void) { return now_nanos(); }

shrike_load_operation *shrike_load_operation_create(void) {
    auto *op = new (std::nothrow) shrike_load_operation();
    if (op) op->submitted = now_nanos();
    return op;
}

void shrike_load_operation_retain(shrike_load_operation *op) {
    if (op) op->references.fetch_add(1, std::memory_order_relaxed);
}

void shrike_load_operation_release(shrike_load_operation *op) {
    if (op && op->references.fetch_sub(1, std::memory_order_acq_rel) == 1) delete op;
}

int shrike_load_operation_state(shrike_load_operation *op) { return op ? state_of(op) : SHRIKE_LOAD_FAILED; }

int shrike_load_operation_mark_in_flight(shrike_load_operation *op) {
    if (!op) return EINVAL;
    std::lock_guard<std::mutex> held(op->lock);
    if (op->state != SHRIKE_LOAD_SUBMITTED) return EALREADY;  // :115-116: started more than once
    op->state = SHRIKE_LOAD_IN_FLIGHT;
    op->started = now_nanos();
    return 0;
}

int shrike_load_operation_finish(shrike_load_operation *op, int failure) {
    if (!op) return EINVAL;
    {
        std::lock_guard<std::mutex> held(op->lock);
        if (terminal(op->state)) return EALREADY;  // :124-125: completed more than once
        op->completed = now_nanos();
        op->state = failure ? SHRIKE_LOAD_FAILED : SHRIKE_LOAD_COMPLETED;
        op->failure = failure;
    }
    op->changed.notify_all();
    return 0;
}

int shrike_load_operation_wait(shrike_load_operation *op) {
    if (!op) return EINVAL;
    std::unique_lock<std::mutex> held(op->lock);
    op->changed.wait(held, [&] { return terminal(op->state); });
    return op->failure;
}

int shrike_load_operation_wait_until(shrike_load_operation *op, uint64_t deadline_nanos) {
    if (!op) return 0;
    std::unique_lock<std::mutex> held(op->lock);
    while (!terminal(op->state)) {
        const uint64_t now = now_nanos();
        if (now >= deadline_nanos) return 0;
        op->changed.wait_for(held, std::chrono::nanoseconds(deadline_nanos - now));
    }
    return 1;
}

uint64_t shrike_load_operation_submitted_nanos(shrike_load_operation *op) { return op ? op->submitted : 0; }

uint64_t shrike_load_operation_started_nanos(shrike_load_operation *op) {
    if (!op) return 0;
    std::lock_guard<std::mutex> held(op->lock);
    return op->started;
}

uint64_t shrike_load_operation_completed_nanos(shrike_load_operation *op) {
    if (!op) return 0;
    std::lock_guard<std::mutex> held(op->lock);
    return op->completed;
}

shrike_prefetch_ring *shrike_prefetch_ring_create(const int *cells, size_t count, shrike_prefetch_drop drop, void *drop_context,
                                                  int *out_errno) {
    auto fail = [&](int err) -> shrike_prefetch_ring * {
        if (out_errno) *out_errno = err;
        return nullptr;
    };
    if (out_errno) *out_errno = 0;
    if (!cells || count == 0) return fail(EINVAL);  // :96-98: invalid prefetch ring geometry
    for (size_t i = 0; i < count; ++i)
        if (contains(cells, i, cells[i])) return fail(EINVAL);
    auto *ring = new (std::nothrow) shrike_prefetch_ring();
    if (!ring) return fail(ENOMEM);
    ring->slots.resize(count);
    for (size_t i = 0; i < count; ++i) ring->slots[i].cell = cells[i];
    ring->drop = drop;
    ring->drop_context = drop_context;
    return ring;
}

void shrike_prefetch_ring_destroy(shrike_prefetch_ring *ring) {
    if (!ring) return;
    for (Slot &slot : ring->slots) ring->attach(slot, nullptr);
    delete ring;
}

int shrike_prefetch_ring_begin(shrike_prefetch_ring *ring, int layer, const int *experts, size_t expert_count, const int *resident,
                               size_t resident_count, int deferred, shrike_prefetch_issue issue, void *issue_context) {
    if (!ring || !issue || (expert_count && !experts) || (resident_count && !resident)) return EINVAL;
    const uint64_t started = now_nanos();
    std::unique_lock<std::mutex> held(ring->lock);
    auto finish = [&](int code) {  // :110-114: the wall of every begin is accounted
        ring->stats.begin_nanos += now_nanos() - started;
        return code;
    };
    ring->reclaim_terminal(layer);
    std::vector<int> wanted;
    for (size_t i = 0; i < expert_count; ++i) {  // :117-123
        const int e = experts[i];
        bool active = false;
        for (const Slot &slot : ring->slots) active |= slot.layer == layer && slot.expert >= 0 && slot.expert == e;
        if (contains(resident, resident_count, e) || active || contains(wanted.data(), wanted.size(), e)) continue;
        wanted.push_back(e);
    }
    std::vector<size_t> free_slots;
    for (size_t i = 0; i < ring->slots.size(); ++i)
        if (ring->slots[i].expert < 0) free_slots.push_back(i);
    const int budget_left = SHRIKE_PREFETCH_IN_FLIGHT_BUDGET - ring->in_flight_count();
    size_t count = wanted.size() < free_slots.size() ? wanted.size() : free_slots.size();
    if (count > size_t(budget_left > 0 ? budget_left : 0)) count = size_t(budget_left > 0 ? budget_left : 0);
    ring->stats.refused += wanted.size() - count;
    if (count == 0) return finish(0);
    std::vector<int> chosen_experts(wanted.begin(), wanted.begin() + long(count)), cells(count);
    for (size_t i = 0; i < count; ++i) {
        Slot &slot = ring->slots[free_slots[i]];
        cells[i] = slot.cell;
        slot.layer = layer;
        slot.expert = chosen_experts[i];
        ring->attach(slot, nullptr);
    }
    held.unlock();
    shrike_load_operation *operation = nullptr;
    int code = issue(issue_context, chosen_experts.data(), cells.data(), count, &operation);
    if (code == 0 && !operation) code = EINVAL;
    held.lock();
    if (code == 0) {
        for (size_t i = 0; i < count; ++i) ring->attach(ring->slots[free_slots[i]], operation);
        ring->stats.issued += count;
        if (deferred) ++ring->stats.deferred;
        return finish(0);
    }
    for (size_t i = 0; i < count; ++i) ring->clear(ring->slots[free_slots[i]]);  // :150-155
    if (code == SHRIKE_PREFETCH_CLAIM_REFUSED) {  // the pool already holds an expert: counted, not an error
        ring->stats.refused += count;
        return finish(0);
    }
    return finish(code);
}

size_t shrike_prefetch_ring_ready_cells(shrike_prefetch_ring *ring, int layer, const int *experts, size_t expert_count,
                                        uint64_t join_nanos, int *out_experts, int *out_cells) {
    if (!ring || (expert_count && !experts) || !out_experts || !out_cells) return 0;
    const uint64_t deadline = join_nanos > 0 ? now_nanos() + join_nanos : 0;
    std::unique_lock<std::mutex> held(ring->lock);
    size_t found = 0;
    std::vector<shrike_load_operation *> joined_ops, late_ops;  // one operation carries a batch (:178-180)
    auto among = [](const std::vector<shrike_load_operation *> &ops, shrike_load_operation *op) {
        for (shrike_load_operation *o : ops)
            if (o == op) return true;
        return false;
    };
    for (size_t index = 0; index < ring->slots.size(); ++index) {
        Slot &slot = ring->slots[index];
        if (slot.layer != layer || !contains(experts, expert_count, slot.expert)) continue;
        if (ring->in_flight(slot)) {
            shrike_load_operation *operation = attached_operation(ring, held, index);
            if (!operation) {
                ++ring->stats.late;
                continue;
            }
            held.unlock();
            const bool joined = deadline > 0 && shrike_load_operation_wait_until(operation, deadline) != 0;
            if (!joined) (void)shrike_load_operation_wait(operation);
            held.lock();
            (joined ? joined_ops : late_ops).push_back(operation);
            shrike_load_operation_release(operation);  // compared by address only from here on
            if (slot.layer != layer || !contains(experts, expert_count, slot.expert)) continue;
        }
        if (!slot.operation) continue;
        if (among(joined_ops, slot.operation)) ++ring->stats.joined;
        else if (among(late_ops, slot.operation)) ++ring->stats.late;
        if (state_of(slot.operation) == SHRIKE_LOAD_COMPLETED) {
            out_experts[found] = slot.expert;
            out_cells[found] = slot.cell;
            ++found;
            slot.leased = true;
        }
    }
    return found;
}

void shrike_prefetch_ring_consume(shrike_prefetch_ring *ring, int layer, const int *experts, size_t expert_count,
                                  const int *freed_experts, const int *freed_cells, size_t freed_count) {
    if (!ring) return;
    std::lock_guard<std::mutex> held(ring->lock);
    for (Slot &slot : ring->slots) {  // :232-252
        if (slot.layer != layer || !contains(experts, expert_count, slot.expert)) continue;
        bool moved = false;
        for (size_t i = 0; i < freed_count && !moved; ++i) {
            if (freed_experts[i] == slot.expert) {
                slot.cell = freed_cells[i];
                moved = true;
            }
        }
        if (!moved && ring->drop) ring->drop(ring->drop_context, layer, slot.expert, slot.cell);
        if (!slot.demand) ++ring->stats.adopted;
        ring->clear(slot);
        slot.leased = false;
        slot.demand = false;
    }
}

size_t shrike_prefetch_ring_claim_demand(shrike_prefetch_ring *ring, int layer, const int *experts, size_t expert_count,
                                         int *out_experts, int *out_cells) {
    if (!ring || (expert_count && !experts) || !out_experts || !out_cells) return 0;
    std::lock_guard<std::mutex> held(ring->lock);
    ring->reclaim_terminal(layer);
    size_t found = 0;
    for (size_t i = 0; i < expert_count; ++i) {  // :257-282
        const int expert = experts[i];
        Slot *own = nullptr;
        for (Slot &slot : ring->slots)
            if (!own && slot.layer == layer && slot.expert == expert) own = &slot;
        if (own) {  // the layer's own failed entry is reused; one still in flight is left to the join
            if (own->leased || !own->operation || state_of(own->operation) != SHRIKE_LOAD_FAILED) continue;
            ++ring->stats.failed;
            ring->attach(*own, nullptr);
        } else {
            for (Slot &slot : ring->slots)
                if (!own && slot.expert < 0) own = &slot;
            if (!own) break;
            own->layer = layer;
            own->expert = expert;
            ring->attach(*own, nullptr);
        }
        own->leased = true;
        own->demand = true;
        out_experts[found] = expert;
        out_cells[found] = own->cell;
        ++found;
    }
    const uint64_t leased = uint64_t(ring->leased_count());
    if (leased > ring->stats.leased_peak) ring->stats.leased_peak = leased;
    return found;
}

void shrike_prefetch_ring_attach_demand(shrike_prefetch_ring *ring, int layer, const int *experts, size_t expert_count,
                                        shrike_load_operation *operation) {
    if (!ring) return;
    std::lock_guard<std::mutex> held(ring->lock);
    for (Slot &slot : ring->slots)
        if (slot.demand && slot.layer == layer && contains(experts, expert_count, slot.expert)) ring->attach(slot, operation);
}

size_t shrike_prefetch_ring_completion_nanos(shrike_prefetch_ring *ring, int layer, const int *experts, size_t expert_count,
                                             int *out_experts, uint64_t *out_nanos) {
    if (!ring || !out_experts || !out_nanos) return 0;
    std::lock_guard<std::mutex> held(ring->lock);
    size_t found = 0;
    for (Slot &slot : ring->slots) {
        if (slot.layer != layer || !contains(experts, expert_count, slot.expert) || !slot.operation) continue;
        if (state_of(slot.operation) != SHRIKE_LOAD_COMPLETED) continue;
        out_experts[found] = slot.expert;
        out_nanos[found] = shrike_load_operation_completed_nanos(slot.operation);
        ++found;
    }
    return found;
}

void shrike_prefetch_ring_unlease(shrike_prefetch_ring *ring, int layer, const int *experts, size_t expert_count) {
    if (!ring) return;
    std::lock_guard<std::mutex> held(ring->lock);
    for (Slot &slot : ring->slots)
        if (slot.layer == layer && contains(experts, expert_count, slot.expert)) slot.leased = false;
}

void shrike_prefetch_ring_note_demand_submission(shrike_prefetch_ring *ring) {
    if (!ring) return;
    std::lock_guard<std::mutex> held(ring->lock);
    if (ring->in_flight_count() > 0) ++ring->stats.overlapped;
}

int shrike_prefetch_ring_note_hook_failure(shrike_prefetch_ring *ring) {
    if (!ring) return 0;
    std::lock_guard<std::mutex> held(ring->lock);
    return ++ring->stats.hook_failures == 1 ? 1 : 0;
}

void shrike_prefetch_ring_statistics(shrike_prefetch_ring *ring, shrike_prefetch_statistics *out) {
    if (!ring || !out) return;
    std::lock_guard<std::mutex> held(ring->lock);
    *out = ring->stats;
}

int shrike_prefetch_ring_in_flight_count(shrike_prefetch_ring *ring) {
    if (!ring) return 0;
    std::lock_guard<std::mutex> held(ring->lock);
    return ring->in_flight_count();
}

int shrike_prefetch_ring_leased_count(shrike_prefetch_ring *ring) {
    if (!ring) return 0;
    std::lock_guard<std::mutex> held(ring->lock);
    return ring->leased_count();
}

}  // extern "C"
