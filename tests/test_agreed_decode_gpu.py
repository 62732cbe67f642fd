"""Decode over a pool of fewer slots than experts with a prefetch ring beside it: a run of tokens, each
with predictions for the next (some right, some wrong, some none), gives for every token the bytes of the
layer with every expert resident, whichever way each selected expert reached HBM: a pool hit, a landed
prediction, a demand read into a ring cell, or an overflow slot."""
import time

import numpy as np
import pytest

from shrike_amd import capi, host
from shrike_amd import synth as S
from harness import runners
from tests.helpers import Layer
from tests.test_decode_gpu import DeviceLayer

pytestmark = pytest.mark.gpu


def wait_for_the_ring(ring, seconds=10.0):
    """The speculative reads issued so far have landed (or failed): what the next token's classifier sees does
    not hang on how fast the storage thread runs."""
    deadline = time.monotonic() + seconds
    while ring.in_flight_count and time.monotonic() < deadline:
        time.sleep(0.0005)
    assert ring.in_flight_count == 0, "a speculative read is still in flight"


def token_inputs(L, count):
    tree = L.tree
    return [(S.f32_to_f16_bits(tree.key(f"agreed.x.{i}").normal(L.d, std=1.0)),
             S.f32_to_f16_bits(tree.key(f"agreed.hidden.{i}").normal(L.d, std=1.0))) for i in range(count)]


@pytest.mark.parametrize("bits,slots,ring_cells,foresight", [(4, 10, 4, 0.75), (8, 8, 2, 0.5), (4, 9, 3, 0.0)])
def test_agreed_layer_with_a_prefetch_ring_equals_the_resident_layer(gpu, bits, slots, ring_cells, foresight):
    d, f, ne, k, tokens = 512, 256, 32, 8, 10
    L = Layer(0x5EED0091 + bits + slots, d, f, ne, k, bits=bits)
    inputs = token_inputs(L, tokens)

    # every token over the layer with all experts resident: the bytes to match, and the routes to foresee
    full = DeviceLayer(gpu, L)
    want = []
    for x, hidden in inputs:
        full.x.upload(x)
        full.hidden.upload(hidden)
        full.moe.encode_decode_layer(full.layer_args())
        gpu.synchronize()
        want.append((full.out_idx.download(np.uint32, k).tolist(), full.y.download(np.uint16, d),
                     full.hidden.download(np.uint16, d)))

    small = DeviceLayer(gpu, L, cells=slots + ring_cells, resident=[])
    small.moe.stream = gpu.Stream()
    arena = host.CellArena(slots + ring_cells)
    cache = host.SlotCache(slots, ne, 0, arena=arena)
    store = gpu.PinnedBuffer(ne * L.stride)
    for e in range(ne):
        store.array[e * L.stride:(e + 1) * L.stride] = L.blobs[e]
    scheduler = host.ExpertIOScheduler(2)
    holder = {}
    ring = host.ExpertPrefetchRing(list(range(slots, slots + ring_cells)),
                                   drop=lambda layer, expert, cell: holder["layer"].drop_landing(layer, expert, cell))
    layer = runners.AgreedDecodeLayer(small.moe, small.pool, cache, ring, small.off, store, L.stride, L.stride, scheduler,
                                  layer=3)
    holder["layer"] = layer
    router = dict(weights=small.router_w, eff_scale=small.eff_scale, expert_scale=small.expert_scale, bias=small.logit_bias)
    residual = gpu.dev(np.zeros(d, np.uint16))  # no shared expert: the fused layer's residual is zero
    rng = np.random.default_rng(bits * 100 + slots)

    try:
        for i, (x, hidden) in enumerate(inputs):
            small.x.upload(x)
            small.hidden.upload(hidden)
            plan = layer.run(router, small.x, residual, small.y, small.hidden)
            small.moe.stream.synchronize()
            idx, y, hid = want[i]
            assert layer.idx.download(np.uint32, k).tolist() == idx, f"token {i}: routes"
            assert np.array_equal(small.y.download(np.uint16, d), y), f"token {i}: y"
            assert np.array_equal(small.hidden.download(np.uint16, d), hid), f"token {i}: hidden"
            # after the plan every selected expert is the pool's, at the cell its entry names
            assert plan.misses == [] and sorted(plan.experts) == sorted(idx)
            for e, cell in zip(plan.experts, plan.assigned_cells):
                assert cache.entry(e) == capi.RESIDENT << 32 | cell and cache.owns_cell(cell)
            assert [small.pool.entry(e) for e in range(ne)] == [cache.entry(e) for e in range(ne)]
            assert ring.leased_count == 0
            # the cells are a partition: the pool's slots and the ring's cells never overlap
            pool_cells = sorted(cache.slot_cell(s) for s in range(slots))
            assert len(set(pool_cells)) == slots and all(0 <= c < slots + ring_cells for c in pool_cells)
            if i + 1 < tokens:
                coming = want[i + 1][0]
                right = [e for e in coming if rng.random() < foresight]
                wrong = [int(e) for e in rng.choice(ne, 2, replace=False) if e not in coming]
                # the next layer's begin comes first in a model: it reclaims this layer's finished landings
                # that no route wanted, so the ring's cells come free again
                ring.begin(4, [], issue=lambda experts, cells: None)
                layer.prefetch(right + wrong)
                wait_for_the_ring(ring)
    finally:
        scheduler.close()

    st, ring_st = cache.statistics(L.stride), ring.statistics
    assert st.loading_slots == 0 and st.pinned_slots == 0
    assert st.requested_experts == tokens * k
    assert layer.fixups >= 1  # the first token finds an empty pool
    assert layer.demand_reads == st.misses
    if foresight == 0.0:
        assert layer.landed_hits == 0
    else:
        assert layer.landed_hits > 0, "no prediction landed ahead of its route"
    assert ring_st["issued"] >= ring_st["adopted"]
    print(f"\nbits {bits} slots {slots} ring {ring_cells}: fixups {layer.fixups}, demand reads {layer.demand_reads}, "
          f"overflow {layer.overflows}, landed hits {layer.landed_hits}, ring {ring_st}")


def test_two_layers_share_one_arena_and_one_ring(gpu):
    """The model's shape: one arena of cells (two layers' slot ranges and the ring's cells), a residency table
    and a slot cache per layer, one ring for both. Each layer's begin reclaims the other's finished landings;
    a landing swapped into one layer's pool hands that layer's freed cell to the ring, so cells migrate between
    the layers' ranges while every token of both layers keeps the resident layers' bytes."""
    d, f, ne, k, tokens = 512, 256, 32, 8, 8
    slots, ring_cells = (10, 9), 3
    cells = sum(slots) + ring_cells
    layers = [Layer(0x5EED00A1, d, f, ne, k, bits=4), Layer(0x5EED00A2, d, f, ne, k, bits=4)]
    inputs = [token_inputs(L, tokens) for L in layers]
    # the second layer routes on what the first one routed on (what is between two MoE layers is left out): the
    # first layer's router pair, whose second router is the second layer's, then foresees the second layer's experts
    inputs[1] = [(inputs[0][t][0], inputs[1][t][1]) for t in range(tokens)]
    want = []
    for L, ins in zip(layers, inputs):
        full, rows = DeviceLayer(gpu, L), []
        for x, hidden in ins:
            full.x.upload(x)
            full.hidden.upload(hidden)
            full.moe.encode_decode_layer(full.layer_args())
            gpu.synchronize()
            rows.append((full.out_idx.download(np.uint32, k).tolist(), full.y.download(np.uint16, d),
                         full.hidden.download(np.uint16, d)))
        want.append(rows)

    arena_pool = gpu.ExpertPool(cells, layers[0].stride, ne)
    pools = [arena_pool, arena_pool.layer_view()]
    arena = host.CellArena(cells)
    caches = [host.SlotCache(slots[0], ne, 0, arena=arena), host.SlotCache(slots[1], ne, slots[0], arena=arena)]
    scheduler = host.ExpertIOScheduler(2)
    agreed = []
    ring = host.ExpertPrefetchRing(list(range(sum(slots), cells)),
                                   drop=lambda layer, expert, cell: agreed[layer].drop_landing(layer, expert, cell))
    devs, routers, stores = [], [], []
    stream = gpu.Stream()
    for index, L in enumerate(layers):
        dev = DeviceLayer(gpu, L, resident=[], pool=pools[index])
        dev.moe.stream = stream
        store = gpu.PinnedBuffer(ne * L.stride)
        for e in range(ne):
            store.array[e * L.stride:(e + 1) * L.stride] = L.blobs[e]
        agreed.append(runners.AgreedDecodeLayer(dev.moe, pools[index], caches[index], ring, dev.off, store, L.stride, L.stride,
                                            scheduler, layer=index))
        routers.append(dict(weights=dev.router_w, eff_scale=dev.eff_scale, expert_scale=dev.expert_scale, bias=dev.logit_bias))
        devs.append(dev)
        stores.append(store)
    residual = gpu.dev(np.zeros(d, np.uint16))
    foreseen = []

    try:
        for t in range(tokens):
            for index in (0, 1):
                dev = devs[index]
                x, hidden = inputs[index][t]
                dev.x.upload(x)
                dev.hidden.upload(hidden)
                # MoE.encodeRouterPair: this layer's router and, as the probe, the following layer's over the same x
                agreed[index].run(routers[index], dev.x, residual, dev.y, dev.hidden, probe=routers[1 - index])
                stream.synchronize()
                idx, y, hid = want[index][t]
                assert agreed[index].idx.download(np.uint32, k).tolist() == idx, f"token {t} layer {index}: routes"
                assert np.array_equal(dev.y.download(np.uint16, d), y), f"token {t} layer {index}: y"
                assert np.array_equal(dev.hidden.download(np.uint16, d), hid), f"token {t} layer {index}: hidden"
                assert [pools[index].entry(e) for e in range(ne)] == [caches[index].entry(e) for e in range(ne)]
                # the runner schedules the next layer's predictions while this layer's reads are behind it
                following, at = (1, t) if index == 0 else (0, t + 1)
                if at < tokens:
                    predicted = agreed[index].predicted_next
                    assert len(predicted) == k and all(0 <= e < ne for e in predicted)
                    if index == 0:  # the probe saw the very row the second layer routes on: it names its experts exactly
                        assert sorted(predicted) == sorted(want[1][t][0])
                    foreseen.append(len(set(predicted) & set(want[following][at][0])))
                    agreed[following].prefetch(predicted)
                    wait_for_the_ring(ring)
            owned = [caches[i].slot_cell(s) for i in (0, 1) for s in range(slots[i])]
            assert len(set(owned)) == sum(slots), "two slots name one cell"
            assert ring.leased_count == 0
    finally:
        scheduler.close()

    moved = [sum(1 for s in range(slots[i]) if not (i * slots[0] <= caches[i].slot_cell(s) < slots[0] + i * slots[1]))
             for i in (0, 1)]
    hits = [a.landed_hits for a in agreed]
    print(f"\ntwo layers: experts foreseen by the router pair per step {foreseen}, landed hits {hits}, slots now on cells outside their first range {moved}, "
          f"overflow {[a.overflows for a in agreed]}, ring {ring.statistics}")
    assert sum(hits) > 0 and sum(moved) > 0
    for cache in caches:
        st = cache.statistics()
        assert st.loading_slots == 0 and st.requested_experts == tokens * k


def test_a_failed_agreed_read_leaves_the_cache_and_the_ring_clean(gpu):
    """A demand batch whose copies fail (forced from the host): the layer raises, the landings are dropped,
    the overflow slots emptied and every lease returned; the same token then runs clean."""
    d, f, ne, k, slots, ring_cells = 256, 128, 16, 4, 5, 2
    L = Layer(0x5EED00B1, d, f, ne, k, bits=4)
    full = DeviceLayer(gpu, L)
    full.moe.encode_decode_layer(full.layer_args())
    gpu.synchronize()
    want = (full.out_idx.download(np.uint32, k).tolist(), full.y.download(np.uint16, d), full.hidden.download(np.uint16, d))

    small = DeviceLayer(gpu, L, cells=slots + ring_cells, resident=[])
    small.moe.stream = gpu.Stream()
    cache = host.SlotCache(slots, ne, 0, arena=host.CellArena(slots + ring_cells))
    store = gpu.PinnedBuffer(ne * L.stride)
    for e in range(ne):
        store.array[e * L.stride:(e + 1) * L.stride] = L.blobs[e]
    scheduler = host.ExpertIOScheduler(1)
    holder = {}
    ring = host.ExpertPrefetchRing(list(range(slots, slots + ring_cells)),
                                   drop=lambda layer, expert, cell: holder["layer"].drop_landing(layer, expert, cell))
    layer = runners.AgreedDecodeLayer(small.moe, small.pool, cache, ring, small.off, store, L.stride, L.stride, scheduler)
    holder["layer"] = layer
    router = dict(weights=small.router_w, eff_scale=small.eff_scale, expert_scale=small.expert_scale, bias=small.logit_bias)
    residual = gpu.dev(np.zeros(d, np.uint16))
    copy = layer._copy

    def failing(experts, cells):
        raise OSError(5, "forced read failure")
    try:
        layer._copy = failing
        with pytest.raises(capi.ShrikeError, match="agreed read failed"):
            layer.run(router, small.x, residual, small.y, small.hidden)
        small.moe.stream.synchronize()
        st = cache.statistics()
        assert st.loading_slots == 0 and st.resident_slots == 0 and cache.resident_experts() == []
        assert all(cache.entry(e) >> 32 == capi.EMPTY for e in range(ne))
        assert ring.leased_count == 0 and ring.in_flight_count == 0
        layer._copy = copy
        small.hidden.upload(L.hidden)
        plan = layer.run(router, small.x, residual, small.y, small.hidden)
        small.moe.stream.synchronize()
        assert plan.misses == [] and layer.idx.download(np.uint32, k).tolist() == want[0]
        assert np.array_equal(small.y.download(np.uint16, d), want[1])
        assert np.array_equal(small.hidden.download(np.uint16, d), want[2])
        assert [small.pool.entry(e) for e in range(ne)] == [cache.entry(e) for e in range(ne)]
    finally:
        scheduler.close()
