// Sanitizer driver for the submission service, the completion timeline and the tagged readback: four producers
// submit demand and speculative work that reserves and publishes timeline values out of order while the main
// thread polls readback words a worker writes.
#include <atomic>
#include <cstdio>
#include <thread>
#include <vector>
#include "shrike_host.h"

struct Job {
    shrike_io_timeline *timeline;
    shrike_io_completion_token token;
    std::atomic<int> *done;
};
static void run_job(void *context) {
    Job *job = static_cast<Job *>(context);
    shrike_io_timeline_publish(job->timeline, &job->token, job->token.value % 7 != 0);
    job->done->fetch_add(1);
    delete job;
}
struct Writer {
    uint32_t *words;
    uint32_t tag, count;
};
static void write_words(void *context) {
    Writer *w = static_cast<Writer *>(context);
    for (uint32_t i = w->count; i-- > 0;) __atomic_store_n(w->words + i, shrike_router_readback_word(w->tag, i), __ATOMIC_RELEASE);
}

int main() {
    int err = 0;
    shrike_io_scheduler *scheduler = shrike_io_scheduler_create(4, &err);
    shrike_io_timeline *timeline = shrike_io_timeline_create(nullptr, 64, &err);
    std::atomic<int> done{0};
    const int per_thread = 2000;
    std::vector<std::thread> producers;
    for (int t = 0; t < 4; ++t)
        producers.emplace_back([&, t] {
            for (int i = 0; i < per_thread; ++i) {
                Job *job = new Job{timeline, {}, &done};
                shrike_io_timeline_reserve(timeline, &job->token);
                shrike_io_scheduler_submit(scheduler, (i + t) % 2, run_job, job);
            }
        });
    uint32_t words[42] = {0};
    shrike_router_readback out;
    uint32_t tag = 0;
    for (int round = 0; round < 200; ++round) {
        tag = shrike_router_readback_next_tag(tag);
        Writer w{words, tag, shrike_router_readback_word_count(8)};
        shrike_io_scheduler_submit(scheduler, SHRIKE_IO_DEMAND, write_words, &w);
        if (!shrike_router_readback_poll(words, 8, tag, shrike_monotonic_nanos() + 5000000000ull, &out)) return 1;
    }
    for (auto &p : producers) p.join();
    shrike_io_scheduler_close(scheduler);
    std::printf("jobs %d published %llu\n", done.load(), (unsigned long long)shrike_io_timeline_published(timeline));
    const bool ok = done.load() == 4 * per_thread && shrike_io_timeline_published(timeline) == uint64_t(4 * per_thread);
    shrike_io_scheduler_destroy(scheduler);
    shrike_io_timeline_destroy(timeline);
    return ok ? 0 : 2;
}
