// ASAN/UBSAN/TSAN driver for the slot cache's landings: one planner thread, one storage thread
#include <atomic>
#include <cstdio>
#include <thread>
#include <vector>
#include "shrike_host.h"
int main() {
    int err = 0;
    shrike_cell_arena *arena = shrike_cell_arena_create(8, &err);
    shrike_slot_cache *c = shrike_slot_cache_create_in_arena(arena, 4, 16, 0, SHRIKE_EVICT_SLRU, 0.5, &err);
    std::atomic<bool> stop{false};
    std::thread storage([&] {
        unsigned n = 0;
        while (!stop.load()) {
            ++n;
            int32_t e = int32_t(n % 16);
            int64_t cell = 4 + n % 4;
            uint32_t r1; if (shrike_slot_cache_claim_prefetch(c, &e, &cell, 1, &r1) == 0) {
                if (n % 3) shrike_slot_cache_complete_landing(c, e, cell);
                else shrike_slot_cache_fail_landing(c, e, cell);
                if (n % 5 == 0) shrike_slot_cache_drop_landing(c, e, cell);
            } else {
                for (int32_t x = 0; x < 16; ++x) shrike_slot_cache_drop_landing(c, x, cell);
            }
            int32_t be[2] = {int32_t(n % 16), int32_t((n + 7) % 16)};
            int64_t bc[2] = {4, 5};
            uint32_t refused;
            if (shrike_slot_cache_claim_prefetch(c, be, bc, 2, &refused) == 0) {
                shrike_slot_cache_complete_landing(c, be[0], bc[0]);
                shrike_slot_cache_complete_landing(c, be[1], bc[1]);
            }
        }
    });
    std::vector<int32_t> ex(3), slots(3), fe(3);
    std::vector<uint64_t> gens(3);
    std::vector<uint32_t> misses(3), cells(3), adopted(3), fc(3);
    for (unsigned step = 0; step < 20000; ++step) {
        int32_t want[3] = {int32_t(step % 16), int32_t((step * 5 + 1) % 16), int32_t((step * 3 + 2) % 16)};
        if (want[0] == want[1] || want[1] == want[2] || want[0] == want[2]) continue;
        shrike_expert_cache_plan plan{0, 0, ex.data(), slots.data(), gens.data(), misses.data(), 0, 0, cells.data(), adopted.data(), 0, 0, fe.data(), fc.data()};
        int rc = shrike_slot_cache_plan_with_landings(c, want, 3, 0, nullptr, 0, nullptr, 0, want, 1, want, 3, -1, &plan);
        if (rc) { static int shown = 0; if (shown++ < 3) std::printf("rc %d step %u\n", rc, step); continue; }
        if (step % 4) shrike_slot_cache_complete(c, &plan, 1000, 500);
        else shrike_slot_cache_abandon(c, &plan);
        int32_t prot[2] = {want[0], want[1]};
        int64_t cell = shrike_slot_cache_reserve_overflow_slot(c, int32_t((step + 9) % 16), prot, 2);
        if (cell >= 0) {
            int32_t oe = int32_t((step + 9) % 16);
            shrike_slot_cache_finish_agreed_reads(c, &oe, &cell, 1, step % 7 != 0, 10, 5);
        }
    }
    stop.store(true);
    storage.join();
    shrike_streaming_statistics st;
    shrike_slot_cache_statistics(c, 1, &st);
    std::printf("plans %llu hits %llu evictions %llu reloads %llu\n", (unsigned long long)st.plans, (unsigned long long)st.hits,
                (unsigned long long)st.evictions, (unsigned long long)st.reloads);
    shrike_slot_cache_destroy(c);
    shrike_cell_arena_destroy(arena);
    return 0;
}
