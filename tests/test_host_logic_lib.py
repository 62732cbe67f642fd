"""The library's host logic (C ABI, include/shrike_host.h) against the restatement in
oracle/host_logic.py, which tests/test_host_logic_oracle.py pins to the reference's vectors:
the same reference cases through the C ABI, then seeded random cases compared for equality."""
import numpy as np
import pytest

from oracle import host_logic as H
from shrike_amd import host as L

U = H.U32_MAX


def to_lib_pairs(pairs):
    a = np.zeros(len(pairs), L.PAIR_DTYPE)
    for i, p in enumerate(pairs):
        a[i] = p.as_tuple()
    return a


def assert_same_grouping(lib: L.GroupedRoutes, ref: H.GroupedRoutes):
    assert [tuple(int(v) for v in p) for p in lib.sorted_pairs] == [p.as_tuple() for p in ref.sorted_pairs]
    assert lib.per_expert_offsets.tolist() == ref.per_expert_offsets
    assert lib.per_expert_counts.tolist() == ref.per_expert_counts
    assert [tuple(int(v) for v in g) for g in lib.groups] == ref.groups
    assert [tuple(int(v) for v in t) for t in lib.tiles] == ref.tiles
    assert (lib.max_pairs_per_expert, lib.max_pairs_per_tile, lib.max_live_experts_per_tile) == (
        ref.max_pairs_per_expert, ref.max_pairs_per_tile, ref.max_live_experts_per_tile)


def test_reference_grouping_case():  # PrefillMoEGroupingTests.swift:5-53
    P = H.Pair
    pairs = [P(0, 3, 0, 10), P(0, 1, 1, 11), P(0, 4, 2, 12), P(1, 1, 0, 13), P(1, 3, 1, 14), P(1, 2, 2, 15),
             P(2, 4, 0, 16), P(2, 3, 1, 17), P(2, 1, 2, 18), P(3, 5, 0, 19), P(3, 1, 1, 20), P(3, 4, 2, 21)][::-1]
    g = L.group_token_expert_pairs(to_lib_pairs(pairs), 4, 3, 6, 2)
    assert g.per_expert_offsets.tolist() == [U, 0, 4, 5, 8, 11]
    assert g.per_expert_counts.tolist() == [0, 4, 1, 3, 3, 1]
    assert [tuple(int(v) for v in t) for t in g.tiles] == [(0, 2, 0, 5), (2, 2, 5, 6), (4, 1, 11, 1)]
    assert_same_grouping(g, H.group_token_expert_pairs(pairs, 4, 3, 6, 2))


@pytest.mark.parametrize("seed", range(12))
def test_random_grouping_matches(seed):
    rng = np.random.default_rng(seed)
    t, k, e = int(rng.integers(0, 70)), int(rng.integers(1, 9)), int(rng.integers(8, 257))
    tile = int(rng.integers(1, 17))
    pairs = []
    for tok in range(t):
        for r, ex in enumerate(rng.choice(e, size=k, replace=False)):
            pairs.append(H.Pair(tok, int(ex), r, int(rng.integers(0, 65536))))
    order = rng.permutation(len(pairs))
    shuffled = [pairs[i] for i in order]
    keys = None
    if seed % 3 == 1:
        keys = [int(v) for v in rng.integers(0, 6, size=e)]  # many equal keys: expert id breaks ties
    elif seed % 3 == 2:
        keys = H.expert_sort_keys([int(v) for v in rng.permutation(e)[: e // 2]], e)
    ref = H.group_token_expert_pairs(shuffled, t, k, e, tile, keys)
    lib = L.group_token_expert_pairs(to_lib_pairs(shuffled), t, k, e, tile, keys)
    assert_same_grouping(lib, ref)
    # the permutation is a stable counting sort of the token-major pairs
    assert_same_grouping(L.group_token_expert_pairs(to_lib_pairs(pairs), t, k, e, tile, keys), ref)


def test_grouping_errors_match():
    P = H.Pair
    cases = [
        ([P(0, 0, 0, 1)], dict(query_count=1, top_k=1, num_experts=1, tile_expert_count=17)),
        ([P(0, 2, 0, 1)], dict(query_count=1, top_k=1, num_experts=2, tile_expert_count=1)),
        ([P(0, 0, 0, 1), P(0, 1, 0, 2)], dict(query_count=1, top_k=2, num_experts=2, tile_expert_count=1)),
        ([P(0, 0, 0, 1)], dict(query_count=1, top_k=1, num_experts=2, tile_expert_count=1, expert_sort_keys=[0])),
        ([P(0, 0, 0, 1)], dict(query_count=-1, top_k=1, num_experts=2, tile_expert_count=1)),
        ([P(0, 0, 0, 1)], dict(query_count=1, top_k=0, num_experts=2, tile_expert_count=1)),
        ([P(0, 0, 0, 1)], dict(query_count=1, top_k=1, num_experts=0, tile_expert_count=1)),
        ([P(0, 0, 0, 1)], dict(query_count=2, top_k=1, num_experts=2, tile_expert_count=1)),
        ([P(3, 0, 0, 1)], dict(query_count=1, top_k=1, num_experts=2, tile_expert_count=1)),
        ([P(0, 0, 5, 1)], dict(query_count=1, top_k=1, num_experts=2, tile_expert_count=1)),
    ]
    for pairs, kw in cases:
        with pytest.raises(H.GroupingError) as ref:
            H.group_token_expert_pairs(pairs, **kw)
        with pytest.raises(L.GroupingError) as lib:
            L.group_token_expert_pairs(to_lib_pairs(pairs), **kw)
        assert (lib.value.case, lib.value.values) == (ref.value.case, ref.value.values), kw


def test_make_pairs_matches():
    rng = np.random.default_rng(5)
    idx, w = rng.integers(0, 256, 48), rng.integers(0, 65536, 48)
    lib = L.make_token_expert_pairs(idx, w, 6, 8)
    ref = H.make_token_expert_pairs(idx, w, 6, 8)
    assert [tuple(int(v) for v in p) for p in lib] == [p.as_tuple() for p in ref]
    assert lib.dtype.itemsize == 16  # PrefillRouterTests.swift:12-19


def test_reference_sweep_orders():  # PrefillMoEGroupingTests.swift:248-348
    rows = {90: 9, 91: 7, 92: 5, 93: 3}
    last = {90: 290, 91: 291, 92: 292, 93: 293}
    for i in range(1, 21):
        rows[i], last[i] = 1, i
    resident = [e in (90, 91, 92, 93) for e in range(94)]
    assert L.resident_first_balanced(rows, last, resident, 50, 8) == [
        1, 2, 3, 4, 5, 6, 90, 93, 7, 8, 9, 10, 11, 12, 13, 91, 14, 15, 16, 17, 18, 19, 20, 92]
    assert L.resident_first_balanced({3: 1, 99: 1}, {3: 0, 99: 1}, [False, False, False, True], 128, 8) == [99, 3]
    assert L.expert_sort_keys([3, 99, 5], 9).tolist() == H.expert_sort_keys([3, 99, 5], 9)


@pytest.mark.parametrize("seed", range(20))
def test_random_sweep_order_matches(seed):
    rng = np.random.default_rng(100 + seed)
    e = int(rng.integers(1, 200))
    ids = [int(v) for v in rng.choice(300, size=e, replace=False)]
    rows = {i: int(rng.integers(1, 40)) for i in ids}
    last = {i: int(rng.integers(0, 64)) for i in ids}
    resident = [bool(v) for v in rng.integers(0, 2, size=int(rng.integers(0, 320)))]
    if seed % 5 == 0:
        resident = [False] * 300
    slots, width = int(rng.integers(1, 256)), int(rng.integers(1, 17))
    assert L.resident_first_balanced(rows, last, resident, slots, width) == H.resident_first_balanced(
        rows, last, resident, slots, width)


def lib_waves(ranges, bound, staging, **kw):
    blocks, waves = L.plan_expert_waves(ranges, bound, staging, **kw)
    out = []
    for w in waves:
        bs = [tuple(int(v) for v in b) for b in blocks[int(w["block_start"]): int(w["block_start"]) + int(w["block_count"])]]
        out.append(H.Wave(bs, int(w["padded_rows"]), int(w["tail_rows"])))
    return out, blocks, waves


RANGES = [(0, 0, 40), (1, 40, 32), (2, 72, 5), (3, 77, 3)]


def test_reference_wave_plans():  # PrefillGroupedRoutedMoETests+Execution.swift:382-432, :535-577
    for staging, kw in ((512, {}), (128, {}), (512, dict(tail_tile=32)), (64, dict(tail_tile=32)), (512, dict(row_tile=32))):
        got, blocks, waves = lib_waves(RANGES, [0, 1, 2, 3], staging, **kw)
        assert got == H.plan_expert_waves(RANGES, [0, 1, 2, 3], staging, **kw)
    got, blocks, waves = lib_waves(RANGES, [0, 1, 2, 3], 512, tail_tile=32)
    assert L.row_tile_tables(blocks, waves[0]) == ([0, 0, 1, 2, 3], [0], [1, 2, 3])
    got, blocks, waves = lib_waves(RANGES, [0, 1, 2, 3], 512)
    assert L.row_tile_table(blocks, waves[0]) == [0, 1, 2, 3]
    with pytest.raises(L.PlanError):
        L.plan_expert_waves(RANGES, [0, 1, 2, 3], 96)
    with pytest.raises(L.PlanError):
        L.plan_expert_waves(RANGES, [0, 1, 2], 512)  # expert 3 is not bound
    with pytest.raises(L.PlanError):
        L.plan_expert_waves(RANGES, [0, 1, 2, 3], 512, row_tile=32, tail_tile=32)


@pytest.mark.parametrize("seed", range(20))
def test_random_wave_plans_match(seed):
    rng = np.random.default_rng(200 + seed)
    n = int(rng.integers(1, 40))
    bound = [int(v) for v in rng.permutation(64)[:n]]
    ranges, start = [], 0
    for e in bound:
        c = int(rng.choice([0, 1, 3, 31, 32, 33, 64, 65, 97, 200, 700]))
        ranges.append((e, start, c))
        start += c
    staging = int(rng.choice([64, 128, 512, 1024]))
    mode = seed % 3
    kw = {} if mode == 0 else dict(tail_tile=32) if mode == 1 else dict(row_tile=32)
    got, blocks, waves = lib_waves(ranges, bound, staging, **kw)
    ref = H.plan_expert_waves(ranges, bound, staging, **kw)
    assert got == ref
    for w, rw in zip(waves, ref):
        if mode == 1:
            assert L.row_tile_tables(blocks, w) == H.row_tile_tables(rw)
        else:
            tile = 32 if mode == 2 else 64
            assert L.row_tile_table(blocks, w, tile) == H.row_tile_table(rw, tile)


# ------------------------------------------------------------------------------ slot cache

def test_reference_slot_cache_cases():  # PreadExpertStreamerTests+CachePlanning.swift
    c = L.SlotCache(4, 8)
    c.load([0, 1])
    plan = c.plan([0, 2], avoiding_slots={0, 1})  # :130-154
    assert plan.assigned_slots == [0, 2] and plan.hits == 1 and plan.misses == [1]
    c = L.SlotCache(4, 8)
    c.load([0, 1])
    assert c.plan([0, 2, 3, 4], avoiding_slots={0, 1}) is None  # :156-169
    c = L.SlotCache(2, 8)
    c.load([0, 1]); c.load([0, 2]); c.load([0, 1])  # :246-270
    s = c.statistics(1000)
    assert (s.plans, s.requested_experts, s.hits, s.misses) == (3, 6, 2, 4)
    assert (s.read_operations, s.bytes_read, s.evictions, s.reloads, s.load_batches) == (4, 4000, 2, 1, 3)
    assert sum(s.latency_histogram) == 3 and s.loading_slots == 0
    c = L.SlotCache(2, 8)
    assert [c.load([e]).assigned_slots[0] for e in range(4)] == [0, 1, 0, 1]  # +Reading.swift:26-53


def test_pins_and_abandon():  # :225-244, :320-341
    c = L.SlotCache(2, 8)
    c.load([0, 1])
    resident = c.plan([0, 1])
    c.pin(resident)
    assert c.statistics().pinned_slots == 2 and c.plan([2]) is None
    c.unpin(resident.assigned_slots, resident.assigned_generations)
    assert c.statistics().pinned_slots == 0
    dropped = c.plan([2, 3])
    assert len(dropped.misses) == 2 and c.statistics().loading_slots == 2 and c.plan([0]) is None
    c.abandon(dropped)
    assert c.statistics().loading_slots == 0
    stale = L.SlotCache(2, 8)
    p = stale.load([0, 1])
    stale.load([2, 3])
    with pytest.raises(L.ShrikeError):
        stale.pin(p)


@pytest.mark.parametrize("seed,slru", [(s, s % 2 == 1) for s in range(10)])
def test_random_slot_cache_trace_matches(seed, slru):
    rng = np.random.default_rng(300 + seed)
    slots, experts = int(rng.integers(2, 24)), int(rng.integers(8, 64))
    share = 0.5 if slru else None
    ref, lib = H.SlotCache(slots, experts, first_cell=3, slru_share=share), L.SlotCache(slots, experts, 3, share)
    open_plans, pinned = [], []
    for step in range(400 if seed else 2200):  # the long run crosses the 1,024-plan aging point twice
        op = rng.integers(0, 10)
        if op < 6 or not open_plans:
            k = int(rng.integers(1, min(slots, 8) + 1))
            zipf = np.minimum(experts - 1, rng.zipf(1.3, size=4 * k) - 1)
            want = list(dict.fromkeys(int(v) for v in zipf))[:k]
            avoid = {int(v) for v in rng.integers(0, slots, size=int(rng.integers(0, 3)))} if op == 5 else set()
            prot = [bool(v) for v in rng.integers(0, 2, size=experts)] if op == 4 else None
            rp = ref.plan(want, avoiding_slots=avoid, protected_experts=prot)
            lp = lib.plan(want, avoiding_slots=avoid, protected_experts=prot)
            assert (rp is None) == (lp is None)
            if rp is None:
                continue
            assert (lp.assigned_slots, lp.assigned_generations, lp.misses, lp.hits) == (
                rp.assigned_slots, rp.assigned_generations, rp.misses, rp.hits)
            open_plans.append((rp, lp))
        elif op < 8:
            rp, lp = open_plans.pop(int(rng.integers(0, len(open_plans))))
            ref.complete(rp); lib.complete(lp)
            if rng.integers(0, 4) == 0:
                try:
                    ref.pin(rp)
                    ok = True
                except RuntimeError:
                    ok = False
                if ok:
                    lib.pin(lp)
                    pinned.append((rp, lp))
                else:
                    with pytest.raises(L.ShrikeError):
                        lib.pin(lp)
        elif op == 8:
            rp, lp = open_plans.pop(int(rng.integers(0, len(open_plans))))
            ref.abandon(rp); lib.abandon(lp)
        elif pinned:
            rp, lp = pinned.pop(0)
            ref.unpin(rp.assigned_slots, rp.assigned_generations)
            lib.unpin(lp.assigned_slots, lp.assigned_generations)
        assert [lib.entry(e) for e in range(experts)] == ref.words
        assert lib.resident_experts() == ref.resident_experts()
    s = lib.statistics()
    assert (s.plans, s.requested_experts, s.hits, s.misses, s.evictions, s.reloads, s.read_operations, s.load_batches,
            s.peak_loading_slots) == tuple(ref.stats[k] for k in (
                "plans", "requested", "hits", "misses", "evictions", "reloads", "read_operations", "load_batches", "peak_loading"))
    counts = ref.counts()
    assert (s.resident_slots, s.loading_slots, s.pinned_slots) == (counts["resident"], counts["loading"], counts["pinned"])


def test_publications_drain_in_order():
    c = L.SlotCache(2, 4, first_cell=6)
    p = c.plan([3])
    assert c.drain_publications() == [(3, (H.LOADING << 32) | 6)]
    c.complete(p)
    c.load([1]); c.load([2])
    pubs = dict(c.drain_publications())
    assert pubs[3] == (H.EMPTY << 32) | U and pubs[2] == (H.RESIDENT << 32) | 6 and pubs[1] == (H.RESIDENT << 32) | 7
    assert c.drain_publications() == []
