// Parallel reader for routed-expert blobs on Linux, behind the reference's own C interface
// (sources/ShrikeKernelsC/include/shrike_expert_io.h): `threads` workers, each with a file
// descriptor of its own, serve up to `batch_depth` published batches in publication order;
// a fetch blocks until its own batch has landed. Where the reference asks the Darwin buffer
// cache to stay out of the way (F_NOCACHE), this opens the descriptors with O_DIRECT, and
// like the reference it fails the reader rather than fall back to cached reads.
#include <fcntl.h>
#include <sys/resource.h>
#include <unistd.h>

#include <cerrno>
#include <condition_variable>
#include <cstdint>
#include <mutex>
#include <new>
#include <thread>
#include <vector>

#include "../../include/shrike_host.h"

namespace {

struct Batch {
    const uint32_t *expert_ids = nullptr;  // exactly one of ids / offsets is set while active
    const uint64_t *offsets = nullptr;
    void *const *destinations = nullptr;
    size_t count = 0, next_index = 0, outstanding = 0;
    int first_errno = 0;
    bool active = false;
    uint64_t sequence = 0;
    std::condition_variable done;  // its own submitter only
};

}  // namespace

struct shrike_expert_reader {
    std::vector<int> fds;
    int depth = 1;
    size_t stride = 0;
    std::vector<std::thread> workers;
    std::mutex lock;
    std::condition_variable work_ready, batch_idle;
    bool shutting_down = false;
    uint64_t next_sequence = 0;
    Batch slots[SHRIKE_IO_MAX_BATCHES];
};

namespace {

void views_of(const shrike_expert_reader &r, shrike_expert_batch_slot *views) {
    for (int i = 0; i < r.depth; ++i) {
        views[i].active = r.slots[i].active ? 1 : 0;
        views[i].sequence = r.slots[i].sequence;
        views[i].next_index = r.slots[i].next_index;
        views[i].count = r.slots[i].count;
    }
}

// expert_io.c:104-124: a short read is legal, end of file inside a blob is not.
int read_blob(int fd, void *dst, size_t bytes, uint64_t offset) {
    auto *out = static_cast<unsigned char *>(dst);
    size_t done = 0;
    while (done < bytes) {
        const ssize_t got = pread(fd, out + done, bytes - done, off_t(offset + done));
        if (got > 0) done += size_t(got);
        else if (got == 0) return EIO;
        else if (errno != EINTR) return errno;
    }
    return 0;
}

void serve(shrike_expert_reader *r, int fd) {
    std::unique_lock<std::mutex> held(r->lock);
    for (;;) {
        int claimed = -1;
        for (;;) {
            shrike_expert_batch_slot views[SHRIKE_IO_MAX_BATCHES];
            views_of(*r, views);
            claimed = shrike_expert_reader_claim_slot(views, r->depth);
            if (claimed >= 0 || r->shutting_down) break;
            r->work_ready.wait(held);
        }
        if (claimed < 0) return;
        Batch &slot = r->slots[claimed];
        const size_t index = slot.next_index++;
        const uint64_t offset = slot.offsets ? slot.offsets[index] : uint64_t(slot.expert_ids[index]) * r->stride;
        void *dst = slot.destinations[index];
        held.unlock();
        const int rc = read_blob(fd, dst, r->stride, offset);
        held.lock();
        // the read still counts in its submitter's `outstanding`: the slot cannot have been reaped
        if (rc != 0 && slot.first_errno == 0) slot.first_errno = rc;
        if (--slot.outstanding == 0) slot.done.notify_one();
    }
}

// expert_io.c:86-100: best effort, never lowers a higher soft limit.
void raise_descriptor_limit() {
    static std::once_flag once;
    std::call_once(once, [] {
        rlimit lim;
        if (getrlimit(RLIMIT_NOFILE, &lim) != 0) return;
        if (lim.rlim_cur < lim.rlim_max) {
            lim.rlim_cur = lim.rlim_max;
            (void)setrlimit(RLIMIT_NOFILE, &lim);
        }
    });
}

int submit(shrike_expert_reader *r, const uint32_t *ids, const uint64_t *offsets, void *const *destinations, size_t count) {
    std::unique_lock<std::mutex> held(r->lock);
    int index;
    for (;;) {  // a published batch is its submitter's until that submitter has reaped it
        if (r->shutting_down) return ECANCELED;
        shrike_expert_batch_slot views[SHRIKE_IO_MAX_BATCHES];
        views_of(*r, views);
        index = shrike_expert_reader_free_slot(views, r->depth);
        if (index >= 0) break;
        r->batch_idle.wait(held);
    }
    Batch &slot = r->slots[index];
    slot.expert_ids = ids; slot.offsets = offsets; slot.destinations = destinations;
    slot.count = count; slot.next_index = 0; slot.outstanding = count;
    slot.first_errno = 0; slot.active = true;
    slot.sequence = r->next_sequence++;
    r->work_ready.notify_all();
    slot.done.wait(held, [&] { return slot.outstanding == 0; });
    const int rc = slot.first_errno;
    // empty again: workers block instead of spinning on a consumed batch, the free-slot search finds it
    slot.expert_ids = nullptr; slot.offsets = nullptr; slot.destinations = nullptr;
    slot.count = 0; slot.next_index = 0; slot.active = false;
    r->batch_idle.notify_all();
    return rc;
}

}  // namespace

extern "C" {

int shrike_expert_reader_claim_slot(const shrike_expert_batch_slot *slots, int slot_count) {
    int best = -1;
    for (int i = 0; i < slot_count; ++i) {
        if (!slots[i].active || slots[i].next_index >= slots[i].count) continue;
        if (best < 0 || slots[i].sequence < slots[best].sequence) best = i;
    }
    return best;
}

int shrike_expert_reader_free_slot(const shrike_expert_batch_slot *slots, int slot_count) {
    for (int i = 0; i < slot_count; ++i)
        if (!slots[i].active) return i;
    return -1;
}

void shrike_expert_reader_cancel_slot(shrike_expert_batch_cancel_state *slot) {
    if (slot->next_index >= slot->count) return;
    slot->outstanding -= slot->count - slot->next_index;
    slot->next_index = slot->count;
    if (slot->first_errno == 0) slot->first_errno = ECANCELED;
}

shrike_expert_reader *shrike_expert_reader_create(const char *path, size_t expert_stride, int threads, int batch_depth,
                                                  int bypass_cache, int *out_errno) {
    auto fail = [&](int err) -> shrike_expert_reader * {
        if (out_errno) *out_errno = err;
        return nullptr;
    };
    if (out_errno) *out_errno = 0;
    if (!path || expert_stride == 0) return fail(EINVAL);
    threads = threads < 1 ? 1 : threads > SHRIKE_IO_MAX_THREADS ? SHRIKE_IO_MAX_THREADS : threads;
    batch_depth = batch_depth < 1 ? 1 : batch_depth > SHRIKE_IO_MAX_BATCHES ? SHRIKE_IO_MAX_BATCHES : batch_depth;
    raise_descriptor_limit();
    auto *r = new (std::nothrow) shrike_expert_reader();
    if (!r) return fail(ENOMEM);
    r->stride = expert_stride;
    r->depth = batch_depth;
    auto close_all = [&] {
        for (int fd : r->fds) close(fd);
        delete r;
    };
    for (int i = 0; i < threads; ++i) {
        // bounded memory is a contract: no silent fall-back to cached reads (expert_io.c:216-229)
        const int fd = open(path, O_RDONLY | O_CLOEXEC | (bypass_cache ? O_DIRECT : 0));
        if (fd < 0) {
            const int err = errno;
            close_all();
            return fail(err);
        }
        r->fds.push_back(fd);
    }
    try {
        for (int i = 0; i < threads; ++i) r->workers.emplace_back(serve, r, r->fds[size_t(i)]);
    } catch (...) {  // a partial pool would read at a fraction of the requested rate (expert_io.c:283-303)
        {
            std::lock_guard<std::mutex> held(r->lock);
            r->shutting_down = true;
        }
        r->work_ready.notify_all();
        for (auto &w : r->workers) w.join();
        close_all();
        return fail(EAGAIN);
    }
    return r;
}

void shrike_expert_reader_destroy(shrike_expert_reader *r) {
    if (!r) return;
    {
        std::lock_guard<std::mutex> held(r->lock);
        r->shutting_down = true;
        for (int i = 0; i < r->depth; ++i) {  // let every waiting submitter's predicate come true
            Batch &slot = r->slots[i];
            if (!slot.active) continue;
            shrike_expert_batch_cancel_state cancel = {slot.count, slot.next_index, slot.outstanding, slot.first_errno};
            shrike_expert_reader_cancel_slot(&cancel);
            slot.next_index = cancel.next_index;
            slot.outstanding = cancel.outstanding;
            slot.first_errno = cancel.first_errno;
            slot.done.notify_one();
        }
    }
    r->work_ready.notify_all();
    r->batch_idle.notify_all();
    for (auto &w : r->workers) w.join();
    for (int fd : r->fds) close(fd);
    delete r;
}

int shrike_expert_reader_fetch(shrike_expert_reader *r, const uint32_t *expert_ids, void *const *destinations, size_t count) {
    if (!r || (count > 0 && (!expert_ids || !destinations))) return EINVAL;
    return count == 0 ? 0 : submit(r, expert_ids, nullptr, destinations, count);
}

int shrike_expert_reader_fetch_offsets(shrike_expert_reader *r, const uint64_t *offsets, void *const *destinations,
                                       size_t count) {
    if (!r || (count > 0 && (!offsets || !destinations))) return EINVAL;
    return count == 0 ? 0 : submit(r, nullptr, offsets, destinations, count);
}

int shrike_expert_reader_threads(const shrike_expert_reader *r) { return r ? int(r->workers.size()) : 0; }
int shrike_expert_reader_batch_depth(const shrike_expert_reader *r) { return r ? r->depth : 0; }

}  // extern "C"

// library-internal: the byte count every read of this reader writes to its destination
size_t shrike_expert_reader_stride_internal(const shrike_expert_reader *r) { return r ? r->stride : 0; }

extern "C" {

}  // extern "C"
