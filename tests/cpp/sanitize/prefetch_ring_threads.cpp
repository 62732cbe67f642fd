#include <atomic>
#include <cstdio>
#include <thread>
#include <vector>
#include "shrike_host.h"
static int issue_cb(void *ctx, const int *, const int *, size_t, shrike_load_operation **out) {
    *out = static_cast<shrike_load_operation *>(ctx);
    return 0;
}
static void drop_cb(void *, int, int, int) {}
int main() {
    int cells[4] = {0, 1, 2, 3}, err = 0;
    shrike_prefetch_ring *ring = shrike_prefetch_ring_create(cells, 4, drop_cb, nullptr, &err);
    std::atomic<bool> stop{false};
    std::thread storage([&] {
        int layer = 0;
        while (!stop.load()) {
            ++layer;
            shrike_load_operation *op = shrike_load_operation_create();
            int experts[2] = {layer % 7, (layer + 1) % 7};
            shrike_prefetch_ring_begin(ring, layer, experts, 2, nullptr, 0, 0, issue_cb, op);
            if (shrike_load_operation_state(op) == SHRIKE_LOAD_SUBMITTED) {
                shrike_load_operation_mark_in_flight(op);
                shrike_load_operation_finish(op, layer % 5 ? 0 : 5);
            }
            shrike_load_operation_release(op);
        }
    });
    int all[7] = {0, 1, 2, 3, 4, 5, 6}, oe[8], oc[8];
    for (int layer = 1; layer < 3000; ++layer) {
        size_t n = shrike_prefetch_ring_ready_cells(ring, layer, all, 7, 200000, oe, oc);
        shrike_prefetch_ring_consume(ring, layer, oe, n, nullptr, nullptr, 0);
        int e8 = 8;
        n = shrike_prefetch_ring_claim_demand(ring, layer, &e8, 1, oe, oc);
        shrike_prefetch_ring_consume(ring, layer, oe, n, nullptr, nullptr, 0);
    }
    stop = true;
    storage.join();
    shrike_prefetch_statistics st;
    shrike_prefetch_ring_statistics(ring, &st);
    printf("issued %llu adopted %llu reclaimed %llu leased %d\n", (unsigned long long)st.issued, (unsigned long long)st.adopted,
           (unsigned long long)st.reclaimed, shrike_prefetch_ring_leased_count(ring));
    shrike_prefetch_ring_destroy(ring);
}
