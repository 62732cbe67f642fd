"""Landings and overflow slots of the slot cache, case by case as the reference's
PreadExpertStreamerTests+Landing.swift holds them (tests/Shrike/Core/Infrastructure/Streaming/),
run against the library and against the oracle's restatement, then the two against each other
on random operation sequences. The cases' file reads and Metal events are outside this layer: a
read is its claim followed by its completion, and `cell(of: plan, index:)` is the plan's
assigned cell."""
import random

import pytest

from oracle import host_logic as H
from shrike_amd import capi
from shrike_amd import host as L

NUM_EXPERTS = 4  # PreadExpertStreamerTests.numExperts
EMPTY_WORD = 0xFFFFFFFF  # ExpertResidencyEntry.notResidentSlot under state 0


def resident(cell):
    return capi.RESIDENT << 32 | cell


def loading(cell):
    return capi.LOADING << 32 | cell


class Fixture:
    """makeLanded: an arena of slot_count + 2 cells (or arena_cells), the last two the ring's."""

    def __init__(self, kind, slot_count=4, first_cell=0, arena_cells=None, slru_share=None):
        cells = arena_cells or slot_count + 2
        if kind == "library":
            self.arena = L.CellArena(cells)
            self.cache = L.SlotCache(slot_count, NUM_EXPERTS, first_cell, slru_share, arena=self.arena)
            self.refused = L.PrefetchClaimRefused
            self.invalid = L.ShrikeError
        else:
            self.arena = H.CellArena(cells)
            self.cache = H.SlotCache(slot_count, NUM_EXPERTS, first_cell, slru_share, arena=self.arena)
            self.refused = H.ClaimRefusedByPool
            self.invalid = ValueError
        self.kind = kind
        self.ring_cells = [cells - 2, cells - 1]

    def word(self, expert):
        return self.cache.entry(expert) if self.kind == "library" else self.cache.words[expert]

    def table(self):
        return [self.word(e) for e in range(NUM_EXPERTS)]

    def land(self, expert, cell):
        self.cache.claim_prefetch([expert], [cell])
        assert self.cache.complete_landing(expert, cell)

    def stat(self, name):
        if self.kind == "library":
            return getattr(self.cache.statistics(), name)
        return self.cache.stats[{"requested_experts": "requested"}.get(name, name)]

    def loading_slots(self):
        return self.cache.statistics().loading_slots if self.kind == "library" else self.cache.counts()["loading"]


@pytest.fixture(params=["library", "oracle"])
def kind(request):
    return request.param


def test_a_claimed_landing_is_loading_at_its_cell_and_neither_a_hit_nor_a_victim(kind):
    f = Fixture(kind)
    ring = f.ring_cells[0]
    assert f.cache.claim_landing(1, ring)
    assert f.word(1) == loading(ring)
    assert 1 not in f.cache.resident_experts()
    plan = f.cache.plan([1])
    assert plan.misses == [0] and plan.assigned_cells[0] < 4
    f.cache.abandon(plan)
    assert not f.cache.claim_landing(1, f.ring_cells[1])


def test_an_overflow_slot_is_a_victim_of_the_pool_loading_at_its_cell(kind):
    f = Fixture(kind, slot_count=2)
    f.cache.load([0, 1])
    first = f.cache.reserve_overflow_slot(2)
    assert first in (0, 1)
    assert f.word(2) == loading(first)
    assert len(f.cache.resident_experts()) == 1
    evicted = 1 if f.cache.resident_experts() == [0] else 0
    assert f.word(evicted) == EMPTY_WORD
    second = f.cache.reserve_overflow_slot(3)
    assert second is not None and second != first
    assert f.cache.resident_experts() == []
    assert f.cache.reserve_overflow_slot(evicted) is None


def test_the_overflow_victim_is_never_one_of_the_route_it_serves(kind):
    f = Fixture(kind, slot_count=2)
    f.cache.load([0, 1])
    assert f.cache.reserve_overflow_slot(2, protecting=[0, 1]) is None
    assert f.cache.resident_experts() == [0, 1]
    cell = f.cache.reserve_overflow_slot(2, protecting=[0, 5])
    assert f.word(2) == loading(cell)
    assert f.cache.resident_experts() == [0]
    assert f.word(1) == EMPTY_WORD


def test_agreed_reads_land_in_a_ring_cell_and_a_pool_cell(kind):
    f = Fixture(kind, slot_count=2)
    f.cache.load([0, 1])
    ring = f.ring_cells[0]
    assert f.cache.claim_landing(3, ring)
    pool = f.cache.reserve_overflow_slot(2)
    assert pool is not None
    f.cache.finish_agreed_reads([3, 2], [ring, pool], True)
    assert f.word(3) == resident(ring) and f.word(2) == resident(pool)
    assert 2 in f.cache.resident_experts() and 3 not in f.cache.resident_experts()
    assert f.stat("read_operations") == 4
    plan = f.cache.plan([3, 2], leased_landings=[3], misses_counted=2)
    assert plan.misses == [] and 3 in plan.freed_cells
    assert plan.assigned_cells == [ring, pool]
    assert f.stat("misses") == 4 and f.stat("hits") == 0


def test_a_failed_agreed_read_drops_its_landing_and_empties_its_pool_cell(kind):
    f = Fixture(kind, slot_count=2)
    f.cache.load([0, 1])
    ring = f.ring_cells[0]
    assert f.cache.claim_landing(3, ring)
    pool = f.cache.reserve_overflow_slot(2)
    f.cache.finish_agreed_reads([3, 2], [ring, pool], False)
    assert f.word(3) == EMPTY_WORD and f.word(2) == EMPTY_WORD
    assert f.cache.claim_landing(3, ring)
    assert f.cache.reserve_overflow_slot(2) is not None


def test_an_abandoned_overflow_slot_is_empty_again(kind):
    # abandonOverflowSlot, PreadExpertStreamer.swift:980-982: a reserved slot whose read was never issued
    f = Fixture(kind, slot_count=2)
    f.cache.load([0, 1])
    cell = f.cache.reserve_overflow_slot(2)
    f.cache.abandon_overflow_slot(3, cell)  # not the slot's expert: nothing happens
    assert f.word(2) == loading(cell)
    f.cache.abandon_overflow_slot(2, cell)
    assert f.word(2) == EMPTY_WORD and f.loading_slots() == 0
    assert f.cache.plan([2]).assigned_cells == [cell]  # the empty slot is the first victim


def test_a_completed_landing_is_a_hit_that_swaps_its_cell_into_the_pool(kind):
    f = Fixture(kind)
    f.cache.load([0, 2])
    ring = f.ring_cells[0]
    f.land(1, ring)
    assert f.word(1) == resident(ring)
    assert f.cache.resident_experts() == [0, 2]
    plan = f.cache.plan([0, 1, 2], leased_landings=[1])
    assert plan.hits == 3 and plan.misses == [] and plan.adopted == []
    assert plan.assigned_cells[1] == ring
    assert list(plan.freed_cells) == [1] and plan.freed_cells[1] in range(4)
    assert f.word(1) == resident(ring)
    assert f.arena.cell_generation(ring) == plan.assigned_generations[1]
    assert f.cache.resident_experts() == [0, 1, 2]
    f.cache.pin(plan)
    f.cache.unpin(plan.assigned_slots, plan.assigned_generations)
    again = f.cache.plan([1])
    assert again.hits == 1 and again.freed_cells == {} and again.assigned_cells == [ring]


def test_a_completed_landing_the_gpu_missed_is_adopted_and_swapped_the_same(kind):
    f = Fixture(kind)
    f.cache.load([0, 2])
    ring = f.ring_cells[0]
    f.land(1, ring)
    plan = f.cache.plan([0, 1, 2], gpu_missed_experts=[1], leased_landings=[1])
    assert plan.hits == 3 and plan.misses == [] and plan.adopted == [1]
    assert plan.assigned_cells[1] == ring and 1 in plan.freed_cells


def test_the_swap_evicts_the_least_used_resident_when_the_pool_is_full(kind):
    f = Fixture(kind, slot_count=3)
    f.cache.load([0, 2, 3])
    f.cache.load([0, 2])
    victim_cell = f.cache.plan([3]).assigned_cells[0]
    ring = f.ring_cells[0]
    f.land(1, ring)
    plan = f.cache.plan([0, 1, 2], leased_landings=[1])
    assert plan.hits == 3 and plan.freed_cells == {1: victim_cell}
    assert f.cache.resident_experts() == [0, 1, 2]
    assert f.word(3) == EMPTY_WORD


def test_an_unwanted_completed_landing_stays_resident_until_dropped(kind):
    f = Fixture(kind)
    f.cache.load([0, 2])
    ring = f.ring_cells[0]
    f.land(1, ring)
    assert f.cache.plan([0, 2]).freed_cells == {}
    assert f.word(1) == resident(ring)
    f.cache.drop_landing(1, ring)
    assert f.word(1) == EMPTY_WORD
    assert f.cache.resident_experts() == [0, 2]
    assert f.cache.plan([1]).misses == [0]


def test_a_failed_landing_is_empty_and_a_miss_again(kind):
    f = Fixture(kind)
    ring = f.ring_cells[0]
    assert f.cache.claim_landing(1, ring)
    f.cache.fail_landing(1, ring)
    assert f.word(1) == EMPTY_WORD
    assert f.cache.plan([1]).misses == [0]
    with pytest.raises(f.invalid):
        f.cache.claim_prefetch([NUM_EXPERTS], [ring])


def test_a_landing_completing_after_the_pool_loaded_its_expert_is_discarded(kind):
    f = Fixture(kind)
    ring = f.ring_cells[0]
    assert f.cache.claim_landing(1, ring)
    f.cache.load([1])
    pooled = f.word(1)
    assert pooled >> 32 == capi.RESIDENT and (pooled & 0xFFFFFFFF) in range(4)
    assert not f.cache.complete_landing(1, ring)
    assert f.word(1) == pooled
    f.cache.drop_landing(1, ring)
    assert f.word(1) == pooled
    assert f.cache.plan([1]).hits == 1


def test_a_prediction_the_pool_holds_refuses_the_batch(kind):
    f = Fixture(kind)
    f.cache.load([1])
    pooled = f.word(1)
    with pytest.raises(f.refused) as refusal:
        f.cache.claim_prefetch([3, 1], f.ring_cells)
    assert (refusal.value.expert, refusal.value.cell) == (1, f.ring_cells[1])
    assert f.word(1) == pooled
    assert f.word(3) == EMPTY_WORD
    assert f.cache.claim_landing(3, f.ring_cells[0])


def test_a_landing_not_leased_to_the_plan_is_read_into_the_pool_and_dropped_later(kind):
    f = Fixture(kind)
    ring = f.ring_cells[0]
    f.land(1, ring)
    plan = f.cache.plan([0, 1, 2])
    assert plan.misses == [0, 1, 2] and plan.freed_cells == {}
    f.cache.complete(plan)
    pooled = f.word(1)
    assert pooled >> 32 == capi.RESIDENT and (pooled & 0xFFFFFFFF) in range(4)
    f.cache.drop_landing(1, ring)
    assert f.word(1) == pooled
    assert f.cache.claim_landing(3, ring)


def test_a_cell_another_landing_holds_or_the_pool_owns_is_refused(kind):
    f = Fixture(kind)
    ring = f.ring_cells[0]
    assert f.cache.claim_landing(1, ring)
    assert not f.cache.claim_landing(3, ring)
    with pytest.raises(f.invalid):
        f.cache.claim_prefetch([3], [0])
    assert f.word(3) == EMPTY_WORD


def test_residency_entries_name_the_arenas_global_cells(kind):
    f = Fixture(kind, slot_count=4, first_cell=4, arena_cells=10)
    f.cache.load([2])
    cell = f.word(2) & 0xFFFFFFFF
    assert cell in range(4, 8)
    assert f.cache.plan([2]).assigned_cells == [cell]
    assert [f.cache.owns_cell(c) for c in (3, 4, 7, 8)] == [False, True, True, False]


def test_the_freed_cell_is_the_rings_next_landing(kind):
    f = Fixture(kind)
    f.cache.load([0, 2])
    ring = f.ring_cells[0]
    f.land(1, ring)
    freed = f.cache.plan([0, 1, 2], leased_landings=[1]).freed_cells[1]
    assert not f.cache.owns_cell(freed) and f.cache.owns_cell(ring)
    f.land(3, freed)
    assert f.word(3) == resident(freed)
    assert f.cache.resident_experts() == [0, 1, 2]
    assert f.cache.plan([3], leased_landings=[3]).hits == 1


def test_a_landing_the_pool_overtook_is_discarded_at_its_completion(kind):
    f = Fixture(kind)
    ring = f.ring_cells[0]
    assert f.cache.claim_landing(1, ring)
    assert f.arena.cell_generation(ring) == 1
    assert f.table() == [EMPTY_WORD, loading(ring), EMPTY_WORD, EMPTY_WORD]
    f.cache.load([1])
    pool = f.word(1) & 0xFFFFFFFF
    assert pool in range(4)
    assert f.arena.cell_generation(pool) == 2
    assert f.table() == [EMPTY_WORD, resident(pool), EMPTY_WORD, EMPTY_WORD]
    assert not f.cache.complete_landing(1, ring)
    assert f.table() == [EMPTY_WORD, resident(pool), EMPTY_WORD, EMPTY_WORD]
    assert f.arena.cell_generation(ring) == 1
    assert f.cache.claim_landing(3, ring)
    assert f.arena.cell_generation(ring) == 3


def test_a_demand_completion_against_a_bumped_cell_generation_throws(kind):
    f = Fixture(kind, slot_count=1)
    stale = f.cache.plan([1])
    assert stale.assigned_slots == [0] and stale.assigned_generations == [1]
    assert f.table() == [EMPTY_WORD, loading(0), EMPTY_WORD, EMPTY_WORD]
    f.cache.abandon(stale)
    assert f.arena.cell_generation(0) == 1
    assert f.table() == [EMPTY_WORD] * 4
    current = f.cache.plan([2])
    assert current.assigned_slots == [0] and current.assigned_generations == [2]
    assert f.arena.cell_generation(0) == 2
    assert f.table() == [EMPTY_WORD, EMPTY_WORD, loading(0), EMPTY_WORD]
    with pytest.raises(Exception, match="generation changed"):
        f.cache.complete(stale)
    assert f.table() == [EMPTY_WORD, EMPTY_WORD, loading(0), EMPTY_WORD]
    assert f.loading_slots() == 1
    f.cache.complete(current)
    assert f.arena.cell_generation(0) == 2
    assert f.table() == [EMPTY_WORD, EMPTY_WORD, resident(0), EMPTY_WORD]


def test_a_swap_then_an_eviction_of_the_same_slot_publishes_empty_once_at_the_cell(kind):
    f = Fixture(kind, slot_count=2)
    f.cache.load([0, 2])
    ring = f.ring_cells[0]
    f.land(1, ring)
    landed = f.word(1)
    assert f.table() == [resident(0), resident(ring), resident(1), EMPTY_WORD]
    swap = f.cache.plan([0, 1], leased_landings=[1])
    assert swap.hits == 2 and swap.assigned_slots == [0, 1]
    assert swap.freed_cells == {1: 1}
    assert swap.assigned_generations == [1, 3]
    assert f.arena.cell_generation(1) == 4 and f.arena.cell_generation(ring) == 3
    assert f.word(1) == landed
    assert f.table() == [resident(0), resident(ring), EMPTY_WORD, EMPTY_WORD]
    evict = f.cache.plan([3])
    assert evict.assigned_slots == [1] and evict.assigned_generations == [5]
    assert f.arena.cell_generation(ring) == 5
    assert f.table() == [resident(0), EMPTY_WORD, EMPTY_WORD, loading(ring)]
    f.cache.complete(evict)
    assert f.arena.cell_generation(ring) == 5
    assert f.table() == [resident(0), EMPTY_WORD, EMPTY_WORD, resident(ring)]


def test_a_stale_completion_after_a_drop_publishes_nothing(kind):
    f = Fixture(kind)
    ring = f.ring_cells[0]
    assert f.cache.claim_landing(1, ring)
    assert f.arena.cell_generation(ring) == 1
    f.cache.drop_landing(1, ring)
    assert f.table() == [EMPTY_WORD] * 4
    assert f.cache.claim_landing(3, ring)
    assert f.arena.cell_generation(ring) == 2
    assert f.table() == [EMPTY_WORD, EMPTY_WORD, EMPTY_WORD, loading(ring)]
    assert not f.cache.complete_landing(1, ring)
    assert f.table() == [EMPTY_WORD, EMPTY_WORD, EMPTY_WORD, loading(ring)]
    assert f.cache.complete_landing(3, ring)
    assert f.table() == [EMPTY_WORD, EMPTY_WORD, EMPTY_WORD, resident(ring)]
    assert f.arena.cell_generation(ring) == 2


def test_an_entry_is_one_word_with_the_state_above_the_cell(kind):
    f = Fixture(kind)
    assert f.word(0) == EMPTY_WORD
    f.cache.load([2])
    cell = f.word(2) & 0xFFFFFFFF
    assert f.word(2) == capi.RESIDENT << 32 | cell
    ring = f.ring_cells[1]
    assert f.cache.claim_landing(3, ring)
    assert f.word(3) == capi.LOADING << 32 | ring
    f.cache.drop_landing(3, ring)
    assert f.word(3) == EMPTY_WORD


def test_an_overflow_slots_first_hit_ends_its_probation_without_promoting_it(kind):
    # makeExpertCachePlan, PreadExpertStreamer.swift:476-481: under SLRU a hit on a slot filled by
    # reserveOverflowSlot takes it off probation; only the next hit promotes it to protected.
    f = Fixture(kind, slot_count=3, slru_share=0.34)  # one protected slot
    f.cache.load([0, 1])
    f.cache.load([0])  # 0 is protected now
    cell = f.cache.reserve_overflow_slot(2)
    assert cell == 2  # the empty slot
    f.cache.mark_overflow_resident(2, cell)
    f.cache.load([2])  # the probation hit: 2 stays unprotected, 0 keeps the protected slot
    victim = f.cache.plan([3])
    assert victim.misses == [0]
    # unprotected slots hold 1 (used at clock 1) and 2 (used at clock 3): the older goes
    assert victim.assigned_slots == [1]
    f.cache.complete(victim)
    f.cache.load([2])  # the second hit promotes 2 and demotes 0, whose last use becomes this clock
    assert f.cache.load([1]).assigned_slots == [1]  # 3, used a clock earlier than the demoted 0
    assert f.cache.plan([3]).assigned_slots == [0]  # 0 is evictable now; 2 holds the protected slot


def test_two_layers_share_one_arena_and_one_generation_clock(kind):
    arena = (L if kind == "library" else H).CellArena(6)
    make = (L if kind == "library" else H).SlotCache
    a = make(2, NUM_EXPERTS, 0, None, arena=arena)
    b = make(2, NUM_EXPERTS, 2, None, arena=arena)
    assert a.plan([0]).assigned_generations == [1]
    assert b.plan([0]).assigned_generations == [2]
    assert a.plan([1]).assigned_generations == [3]
    assert [arena.cell_generation(c) for c in range(6)] == [1, 3, 2, 0, 0, 0]
    assert b.claim_landing(3, 4) and arena.cell_generation(4) == 4
    assert a.claim_landing(3, 5) and arena.cell_generation(5) == 5  # the layers' landings are their own


def test_creating_a_cache_outside_its_arena_fails():
    arena = L.CellArena(4)
    with pytest.raises(L.ShrikeError):
        L.SlotCache(4, NUM_EXPERTS, 1, arena=arena)
    with pytest.raises(L.ShrikeError):
        L.CellArena(0)
    assert L.SlotCache(4, NUM_EXPERTS, 0, arena=arena).slot_cell(3) == 3


@pytest.mark.parametrize("seed", range(6))
def test_the_library_follows_the_restatement_through_random_landings_and_overflows(seed):
    rng = random.Random(seed)
    slots, experts, ring = rng.choice([2, 3, 5]), rng.choice([6, 9]), 3
    share = rng.choice([None, 0.4])
    ref_arena, lib_arena = H.CellArena(slots + ring + 1), L.CellArena(slots + ring + 1)
    ref = H.SlotCache(slots, experts, 1, share, arena=ref_arena)
    lib = L.SlotCache(slots, experts, 1, share, arena=lib_arena)
    free_ring = list(range(slots + 1, slots + ring + 1))
    landed = {}  # expert -> cell, as the ring would hold them
    open_plans = []

    def same_state():
        assert [lib.entry(e) for e in range(experts)] == ref.words
        assert [lib_arena.cell_generation(c) for c in range(slots + ring + 1)] == ref_arena.generations
        assert lib.resident_experts() == ref.resident_experts()
        assert [lib.slot_cell(s) for s in range(slots)] == ref.slot_cell
        st = lib.statistics()
        assert (st.plans, st.hits, st.misses, st.evictions, st.reloads, st.read_operations, st.load_batches) == tuple(
            ref.stats[k] for k in ("plans", "hits", "misses", "evictions", "reloads", "read_operations", "load_batches"))

    for _ in range(400):
        op = rng.random()
        if op < 0.3:
            wanted = rng.sample(range(experts), rng.randint(1, min(slots, 3)))
            leased = [e for e in wanted if e in landed and rng.random() < 0.8]
            missed = [e for e in wanted if rng.random() < 0.5]
            rp = ref.plan(wanted, gpu_missed_experts=missed, leased_landings=leased)
            lp = lib.plan(wanted, gpu_missed_experts=missed, leased_landings=leased)
            assert (rp is None) == (lp is None)
            if rp is not None:
                assert (lp.assigned_slots, lp.assigned_generations, lp.misses, lp.hits, lp.adopted, lp.freed_cells,
                        lp.assigned_cells) == (rp.assigned_slots, rp.assigned_generations, rp.misses, rp.hits,
                                               rp.adopted, rp.freed_cells, rp.assigned_cells)
                for e, cell in rp.freed_cells.items():
                    free_ring.append(cell)  # the swap: the landing's cell is the pool's, the freed cell the ring's
                    del landed[e]
                open_plans.append((rp, lp))
        elif op < 0.45 and open_plans:
            rp, lp = open_plans.pop(rng.randrange(len(open_plans)))
            if rng.random() < 0.8:
                outcomes = []
                for cache, plan in ((ref, rp), (lib, lp)):
                    try:
                        cache.complete(plan)
                        outcomes.append(True)
                    except Exception:
                        outcomes.append(False)
                assert outcomes[0] == outcomes[1]
            else:
                ref.abandon(rp)
                lib.abandon(lp)
        elif op < 0.6 and free_ring:
            e, cell = rng.randrange(experts), free_ring[-1]
            claimed = ref.claim_landing(e, cell)
            assert lib.claim_landing(e, cell) == claimed
            if claimed:
                free_ring.pop()
                landed[e] = cell
        elif op < 0.75 and landed:
            e = rng.choice(sorted(landed))
            done = ref.complete_landing(e, landed[e])
            assert lib.complete_landing(e, landed[e]) == done
        elif op < 0.85 and landed:
            e = rng.choice(sorted(landed))
            ref.drop_landing(e, landed[e])
            lib.drop_landing(e, landed[e])
            free_ring.append(landed.pop(e))
        elif op < 0.95:
            e = rng.randrange(experts)
            protecting = rng.sample(range(experts), rng.randint(0, 2))
            cell = ref.reserve_overflow_slot(e, protecting)
            assert lib.reserve_overflow_slot(e, protecting) == cell
            if cell is not None:
                if rng.random() < 0.7:
                    ref.finish_agreed_reads([e], [cell], True)
                    lib.finish_agreed_reads([e], [cell], True)
                else:
                    ref.abandon_overflow_slot(e, cell)
                    lib.abandon_overflow_slot(e, cell)
        else:
            batch = rng.sample(range(experts), 2)
            cells = free_ring[-2:]
            if len(cells) == 2:
                outcomes = []
                for cache, refused in ((ref, H.ClaimRefusedByPool), (lib, L.PrefetchClaimRefused)):
                    try:
                        cache.claim_prefetch(batch, cells)
                        outcomes.append(None)
                    except refused as r:
                        outcomes.append((r.expert, r.cell))
                assert outcomes[0] == outcomes[1]
                if outcomes[0] is None:
                    for e, cell in zip(batch, cells):
                        landed[e] = cell
                        free_ring.remove(cell)
        same_state()
