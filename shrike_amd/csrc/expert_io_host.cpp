// Host-side plumbing of the miss protocol that is neither the slot cache nor the reader:
//   * the submission service with two queues (ExpertIOScheduler, ExpertLoadOperation.swift:166-219),
//   * the completion timeline of all expert reads (ExpertIOEventCoordinator.swift:23-90),
//   * the host's half of the classifier's tagged readback (RouterHostReadback.swift:8-63) over acquire loads
//     (sources/ShrikeKernelsC/include/shrike_atomics.h:7-14).
// No device call in this file.
#include <atomic>
#include <condition_variable>
#include <deque>
#include <mutex>
#include <set>
#include <thread>
#include <vector>

#include "../../include/shrike_host.h"
#include "host_common.h"

using shrike::set_error;

// ------------------------------------------------------------------ submission service

struct shrike_io_scheduler {
    struct Item {
        shrike_io_work work;
        void *context;
    };
    std::mutex lock;
    std::condition_variable wake;
    std::deque<Item> queue[2];  // [SHRIKE_IO_DEMAND], [SHRIKE_IO_SPECULATIVE]
    bool closed = false;
    std::vector<std::thread> workers;

    // ExpertIOScheduler.runWorker, ExpertLoadOperation.swift:205-218: a queued demand batch goes first
    void run() {
        for (;;) {
            Item item;
            {
                std::unique_lock<std::mutex> hold(lock);
                wake.wait(hold, [&] { return closed || !queue[0].empty() || !queue[1].empty(); });
                std::deque<Item> &from = queue[0].empty() ? queue[1] : queue[0];
                if (from.empty()) return;  // closed and drained
                item = from.front();
                from.pop_front();
            }
            item.work(item.context);
        }
    }
};

// ------------------------------------------------------------------ completion timeline

struct shrike_io_timeline {
    std::mutex lock;
    uint32_t *status;          // word_count words the consumers read (caller-owned, or `own`)
    std::vector<uint32_t> own;
    uint32_t word_count;
    uint64_t next_value = 1, published = 0;
    std::set<uint64_t> terminal;
};

extern "C" {

shrike_io_scheduler *shrike_io_scheduler_create(int worker_count, int *out_errno) {
    if (worker_count <= 0 || worker_count > 64) {  // ExpertLoadOperation.swift:183: precondition(workerCount > 0)
        set_error("ExpertIOScheduler: workerCount=%d must be in 1...64", worker_count);
        if (out_errno) *out_errno = EINVAL;
        return nullptr;
    }
    auto *s = new shrike_io_scheduler();
    try {
        for (int i = 0; i < worker_count; ++i) s->workers.emplace_back([s] { s->run(); });
    } catch (...) {
        {
            std::lock_guard<std::mutex> hold(s->lock);
            s->closed = true;
        }
        s->wake.notify_all();
        for (auto &t : s->workers) t.join();
        delete s;
        set_error("ExpertIOScheduler: a worker thread could not be started");
        if (out_errno) *out_errno = EAGAIN;
        return nullptr;
    }
    if (out_errno) *out_errno = 0;
    return s;
}

int shrike_io_scheduler_submit(shrike_io_scheduler *scheduler, int priority, shrike_io_work work, void *context) {
    SHRIKE_REQUIRE(scheduler && work, "ExpertIOScheduler.submit: NULL argument");
    SHRIKE_REQUIRE(priority == SHRIKE_IO_DEMAND || priority == SHRIKE_IO_SPECULATIVE, "ExpertIOScheduler.submit: priority %d", priority);
    {
        std::lock_guard<std::mutex> hold(scheduler->lock);
        if (scheduler->closed) {
            set_error("the expert I/O scheduler is closed");
            return ESHUTDOWN;
        }
        scheduler->queue[priority].push_back({work, context});
    }
    scheduler->wake.notify_one();
    return 0;
}

void shrike_io_scheduler_close(shrike_io_scheduler *scheduler) {
    if (!scheduler) return;
    {
        std::lock_guard<std::mutex> hold(scheduler->lock);
        if (scheduler->closed && scheduler->workers.empty()) return;
        scheduler->closed = true;
    }
    scheduler->wake.notify_all();
    for (auto &t : scheduler->workers) t.join();
    scheduler->workers.clear();
}

void shrike_io_scheduler_destroy(shrike_io_scheduler *scheduler) {
    if (!scheduler) return;
    shrike_io_scheduler_close(scheduler);
    delete scheduler;
}

int shrike_io_scheduler_workers(const shrike_io_scheduler *scheduler) { return scheduler ? int(scheduler->workers.size()) : 0; }

// ---- timeline

shrike_io_timeline *shrike_io_timeline_create(uint32_t *status_words, uint32_t word_count, int *out_errno) {
    if (word_count == 0) word_count = SHRIKE_IO_STATUS_WORDS;
    auto *t = new shrike_io_timeline();
    t->word_count = word_count;
    if (status_words) {
        t->status = status_words;
    } else {
        t->own.assign(word_count, 0u);
        t->status = t->own.data();
    }
    if (out_errno) *out_errno = 0;
    return t;
}

void shrike_io_timeline_destroy(shrike_io_timeline *timeline) { delete timeline; }

// ExpertIOEventCoordinator.reserve, ExpertIOEventCoordinator.swift:48-78
int shrike_io_timeline_reserve(shrike_io_timeline *timeline, shrike_io_completion_token *out) {
    SHRIKE_REQUIRE(timeline && out, "ExpertIOEventCoordinator.reserve: NULL argument");
    std::lock_guard<std::mutex> hold(timeline->lock);
    if (timeline->next_value == 0 || timeline->next_value == UINT64_MAX) {
        set_error("internal inconsistency: expert I/O shared-event value space exhausted");
        return ERANGE;
    }
    const uint32_t index = uint32_t((timeline->next_value - 1) % timeline->word_count);
    __atomic_store_n(timeline->status + index, SHRIKE_IO_STATUS_LOADING, __ATOMIC_RELEASE);
    out->value = timeline->next_value++;
    out->status_index = index;
    out->status = timeline->status + index;
    return 0;
}

// ExpertIOEventCoordinator.publish, ExpertIOEventCoordinator.swift:80-89: the status word first, then the
// published value moves over every value whose predecessors are all terminal.
uint64_t shrike_io_timeline_publish(shrike_io_timeline *timeline, const shrike_io_completion_token *token, int succeeded) {
    if (!timeline || !token) return 0;
    std::lock_guard<std::mutex> hold(timeline->lock);
    __atomic_store_n(timeline->status + token->status_index, succeeded ? SHRIKE_IO_STATUS_COMPLETE : SHRIKE_IO_STATUS_FAILED,
                     __ATOMIC_RELEASE);
    timeline->terminal.insert(token->value);
    for (auto it = timeline->terminal.find(timeline->published + 1); it != timeline->terminal.end();
         it = timeline->terminal.find(timeline->published + 1)) {
        timeline->terminal.erase(it);
        ++timeline->published;
    }
    return timeline->published;
}

uint64_t shrike_io_timeline_published(shrike_io_timeline *timeline) {
    if (!timeline) return 0;
    std::lock_guard<std::mutex> hold(timeline->lock);
    return timeline->published;
}

// ---- tagged readback, host side

uint32_t shrike_load_acquire_u32(const uint32_t *word) { return __atomic_load_n(word, __ATOMIC_ACQUIRE); }
void shrike_store_release_u64(uint64_t *word, uint64_t value) { __atomic_store_n(word, value, __ATOMIC_RELEASE); }

uint32_t shrike_router_readback_word_count(uint32_t top_k) { return 2u + 5u * top_k; }
uint32_t shrike_router_readback_word(uint32_t tag, uint32_t value) { return (tag << 16) | (value & 0xffffu); }
uint32_t shrike_router_readback_next_tag(uint32_t tag) { return tag >= 0xffffu ? 1u : tag + 1u; }

int shrike_router_readback_is_complete(const uint32_t *words, uint32_t top_k, uint32_t tag) {
    if (!words) return 0;
    const uint32_t count = shrike_router_readback_word_count(top_k);
    for (uint32_t i = 0; i < count; ++i)
        if (shrike_load_acquire_u32(words + i) >> 16 != tag) return 0;
    return 1;
}

int shrike_router_readback_decode(const uint32_t *words, uint32_t top_k, uint32_t tag, shrike_router_readback *out) {
    if (!words || !out || top_k == 0 || top_k > SHRIKE_MAX_TOP_K) return 0;
    const uint32_t count = shrike_router_readback_word_count(top_k);
    uint32_t values[2 + 5 * SHRIKE_MAX_TOP_K];
    for (uint32_t i = 0; i < count; ++i) {
        const uint32_t word = shrike_load_acquire_u32(words + i);
        if (word >> 16 != tag) return 0;  // RouterHostReadback.swift:47: nil until every word carries the tag
        values[i] = word & 0xffffu;
    }
    shrike_router_readback r = {};
    r.hit_count = values[0] < top_k ? values[0] : top_k;
    r.miss_count = values[1] < top_k ? values[1] : top_k;
    for (uint32_t i = 0; i < top_k; ++i) {
        r.expert_ids[i] = values[2 + i];
        r.weight_bits[i] = uint16_t(values[2 + top_k + i]);
        if (i < r.hit_count) r.hit_positions[i] = values[2 + 2 * top_k + i];
        if (i < r.miss_count) r.miss_positions[i] = values[2 + 3 * top_k + i];
        r.predicted_ids[i] = values[2 + 4 * top_k + i];
    }
    *out = r;
    return 1;
}

int shrike_router_readback_poll(const uint32_t *words, uint32_t top_k, uint32_t tag, uint64_t deadline_nanos,
                                shrike_router_readback *out) {
    for (uint32_t spins = 0;; ++spins) {
        if (shrike_router_readback_decode(words, top_k, tag, out)) return 1;
        if (shrike_monotonic_nanos() >= deadline_nanos) return 0;
        if (spins > 64) std::this_thread::yield();
    }
}

}  // extern "C"
