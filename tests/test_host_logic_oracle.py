"""The host-logic restatement against the vectors the reference's own unit tests hold.

Each test names the reference test it takes its inputs and expected outputs from; nothing
here reads the reference at run time."""
import pytest

from oracle import host_logic as H
from oracle.host_logic import Pair

U = H.U32_MAX


def P(token, expert, rank, bits):
    return Pair(token, expert, rank, bits)


# ------------------------------------------------------------------ budget and ladder
# tests/Shrike/Core/Runtime/Configuration/ExpertCacheBudgetTests.swift

STRIDE4, STRIDE6, STRIDE8, LAYERS = 1_769_472, 2_555_904, 3_342_336, 40


def test_default_budget_per_quant():  # :20-29
    assert H.expert_cache_slots(STRIDE4, LAYERS) == 128
    assert H.expert_cache_slots(STRIDE8, LAYERS) == 64


def test_ladder_membership_and_monotonic():  # :31-53
    for stride in (STRIDE4, STRIDE6, STRIDE8):
        for budget in (1 << 28, 1 << 30, 1 << 32, 1 << 34):
            assert H.expert_cache_slots(stride, LAYERS, budget) in H.ALLOWED_SLOTS
    prev = 0
    for budget in (1 << 27, 1 << 28, 1 << 29, 1 << 30, 1 << 31, 1 << 32):
        s = H.expert_cache_slots(STRIDE4, LAYERS, budget)
        assert s >= prev
        prev = s


def test_degenerate_and_production_budget():  # :66-71, :85-89
    assert H.expert_cache_slots(0, LAYERS) == 8
    assert H.expert_cache_slots(STRIDE4, 0) == 8
    assert H.expert_cache_slots(STRIDE4, LAYERS, 11_324_620_800) == 160


def test_budget_drives_slots():  # :141-153
    assert [H.expert_cache_slots(STRIDE4, 40, g << 30) for g in (1, 4, 8)] == [16, 64, 128]


def test_parse_budget():  # :117-138
    ok = {"8G": 8 << 30, "2g": 2 << 30, "512M": 512 << 20, "8GiB": 8 << 30, "1024KB": 1024 << 10,
          " 4G ": 4 << 30, "1073741824": 1 << 30, "1.5G": int(1.5 * (1 << 30)), "0.5G": 1 << 29}
    for text, want in ok.items():
        assert H.parse_budget_bytes(text) == want, text
    for bad in ["", " ", "bogus", "G", "-2G", "0", "0G", "abcG", "2X", "2GG"]:
        assert H.parse_budget_bytes(bad) is None, bad


# ---------------------------------------------------------------------------- grouping
# tests/Shrike/Core/Kernels/Prefill/PrefillMoEGroupingTests.swift

def test_grouping_sorts_and_builds_tables():  # :5-53
    pairs = [P(0, 3, 0, 10), P(0, 1, 1, 11), P(0, 4, 2, 12), P(1, 1, 0, 13), P(1, 3, 1, 14), P(1, 2, 2, 15),
             P(2, 4, 0, 16), P(2, 3, 1, 17), P(2, 1, 2, 18), P(3, 5, 0, 19), P(3, 1, 1, 20), P(3, 4, 2, 21)][::-1]
    g = H.group_token_expert_pairs(pairs, 4, 3, 6, tile_expert_count=2)
    assert [p.expert for p in g.sorted_pairs] == [1, 1, 1, 1, 2, 3, 3, 3, 4, 4, 4, 5]
    assert [[p.token, p.rank] for p in g.sorted_pairs] == [
        [0, 1], [1, 0], [2, 2], [3, 1], [1, 2], [0, 0], [1, 1], [2, 1], [0, 2], [2, 0], [3, 2], [3, 0]]
    assert g.per_expert_offsets == [U, 0, 4, 5, 8, 11]
    assert g.per_expert_counts == [0, 4, 1, 3, 3, 1]
    assert g.groups == [(1, 0, 4), (2, 4, 1), (3, 5, 3), (4, 8, 3), (5, 11, 1)]
    assert g.tiles == [(0, 2, 0, 5), (2, 2, 5, 6), (4, 1, 11, 1)]
    assert (g.max_pairs_per_expert, g.max_pairs_per_tile, g.max_live_experts_per_tile) == (4, 6, 2)


def test_grouping_order_independent_and_keeps_weight_bits():  # :55-82
    tm = [P(0, 2, 0, 101), P(0, 1, 1, 102), P(1, 2, 0, 103), P(1, 0, 1, 104), P(2, 1, 0, 105), P(2, 2, 1, 106)]
    sh = [tm[5], tm[1], tm[3], tm[0], tm[4], tm[2]]
    a = H.group_token_expert_pairs(tm, 3, 2, 3, 2)
    b = H.group_token_expert_pairs(sh, 3, 2, 3, 2)
    assert a == b
    assert [p.weight_bits for p in a.sorted_pairs] == [104, 102, 105, 101, 103, 106]


def test_grouping_by_sort_keys():  # :84-115
    pairs = [P(0, 1, 0, 10), P(0, 2, 1, 20), P(1, 3, 0, 30), P(1, 1, 1, 11), P(2, 2, 0, 21), P(2, 3, 1, 31)]
    g = H.group_token_expert_pairs(pairs, 3, 2, 4, 2, expert_sort_keys=[0, 30, 10, 20])
    assert [x[0] for x in g.groups] == [2, 3, 1]
    assert [p.expert for p in g.sorted_pairs] == [2, 2, 3, 3, 1, 1]
    assert g.per_expert_offsets == [U, 4, 0, 2]
    assert g.tiles == [(0, 2, 0, 4), (2, 1, 4, 2)]


def test_grouping_rejections():  # :117-173
    with pytest.raises(H.GroupingError) as e:
        H.group_token_expert_pairs([P(0, 0, 0, 1)], 1, 1, 1, 17)
    assert (e.value.case, e.value.values) == ("invalidTileExpertCount", (17,))
    with pytest.raises(H.GroupingError) as e:
        H.group_token_expert_pairs([P(0, 2, 0, 1)], 1, 1, 2, 1)
    assert (e.value.case, e.value.values) == ("expertOutOfRange", (2,))
    with pytest.raises(H.GroupingError) as e:
        H.group_token_expert_pairs([P(0, 0, 0, 1), P(0, 1, 0, 2)], 1, 2, 2, 1)
    assert (e.value.case, e.value.values) == ("duplicateTokenRank", (0, 0))
    with pytest.raises(H.GroupingError) as e:
        H.group_token_expert_pairs([P(0, 0, 0, 1)], 1, 1, 2, 1, expert_sort_keys=[0])
    assert (e.value.case, e.value.values) == ("expertSortKeyCountMismatch", (2, 1))


def test_grouping_trace_pressure():  # :175-203
    pairs = [P(t, (t + r * 7) % 74, r, t * 8 + r) for t in range(32) for r in range(8)]
    g = H.group_token_expert_pairs(pairs, 32, 8, 128, 16)
    assert len(g.sorted_pairs) == 256 and len(g.groups) <= 74
    assert g.max_live_experts_per_tile <= 16 and g.max_pairs_per_tile <= 256
    assert all(t[1] <= 16 and t[3] > 0 for t in g.tiles)


def test_grouping_by_sweep_order():  # :205-229
    pairs = [P(0, 8, 0, 80), P(1, 3, 0, 10), P(2, 8, 0, 81), P(3, 5, 0, 50)]
    keys = H.expert_sort_keys([3, 8, 5], 9)
    g = H.group_token_expert_pairs(pairs, 4, 1, 9, 2, expert_sort_keys=keys)
    assert [x[0] for x in g.groups] == [3, 8, 5]
    assert [p.expert for p in g.sorted_pairs] == [3, 8, 8, 5]
    assert g.tiles == [(0, 2, 0, 3), (2, 1, 3, 1)]


def test_expert_sort_keys():  # :231-246
    keys = H.expert_sort_keys([3, 8, 5], 9)
    assert (keys[3], keys[8], keys[5]) == (0, 1, 2)
    assert all(keys[e] == 3 for e in (0, 1, 2, 4, 6, 7))
    keys = H.expert_sort_keys([3, 99, 5], 9)
    assert len(keys) == 9 and keys[3] == 0 and keys[5] == 2


def test_resident_first_balanced_spread():  # :248-268
    rows = {90: 9, 91: 7, 92: 5, 93: 3}
    last = {90: 290, 91: 291, 92: 292, 93: 293}
    for i in range(1, 21):
        rows[i], last[i] = 1, i
    resident = [False] * 94
    for e in (90, 91, 92, 93):
        resident[e] = True
    order = H.resident_first_balanced(rows, last, resident, 50, 8)
    assert order == [1, 2, 3, 4, 5, 6, 90, 93, 7, 8, 9, 10, 11, 12, 13, 91, 14, 15, 16, 17, 18, 19, 20, 92]


def _head_case():
    rows, last = {}, {}
    for i in range(1, 10):
        rows[i], last[i] = 1, 9 + i
    for i in range(100, 103):
        rows[i], last[i] = 1, i - 100
    resident = [False] * 103
    for i in range(1, 10):
        resident[i] = True
    return rows, last, resident


def test_resident_first_balanced_head():  # :270-289
    rows, last, resident = _head_case()
    assert H.resident_first_balanced(rows, last, resident, 20, 8) == [1, 2, 3, 4, 5, 6, 7, 8, 100, 101, 102, 9]


def test_resident_first_balanced_exhausted_head():  # :291-307
    rows, last = {999: 1}, {999: 0}
    for i in range(1, 101):
        rows[i], last[i] = 1, i
    resident = [False] * 1000
    resident[999] = True
    order = H.resident_first_balanced(rows, last, resident, 1, 8)
    assert set(order) == set(rows) and len(order) == 101


def test_resident_first_balanced_small_cases():  # :309-348
    resident = [False] * 10
    resident[3] = resident[7] = True
    assert H.resident_first_balanced({3: 1, 5: 1}, {3: 0, 5: 1}, resident, 128, 8) == [5, 3]
    assert H.resident_first_balanced({3: 1, 99: 1}, {3: 0, 99: 1}, [False, False, False, True], 128, 8) == [99, 3]
    long_res = [False] * 200
    long_res[5] = True
    assert H.resident_first_balanced({2: 3, 5: 1}, {2: 4, 5: 1}, long_res, 128, 8) == [2, 5]


def test_grouping_reproduces_sweep_tiles():  # :350-388
    rows, last, resident = _head_case()
    pairs = [P(i - 1, i, 0, i) for i in range(1, 10)] + [P(i - 91, i, 0, i) for i in range(100, 103)]
    order = H.resident_first_balanced(rows, last, resident, 20, 8)
    g = H.group_token_expert_pairs(pairs, 12, 1, 103, 8, expert_sort_keys=H.expert_sort_keys(order, 103))
    assert [x[0] for x in g.groups] == order
    assert g.tiles == [(0, 8, 0, 8), (8, 4, 8, 4)]


def test_pairs_token_major():  # PrefillRouterTests layout: token, expert, rank, weight bits
    pairs = H.make_token_expert_pairs([5, 2, 7, 1], [0x3C00, 0x3800, 0x3400, 0x3000], 2, 2)
    assert [p.as_tuple() for p in pairs] == [(0, 5, 0, 0x3C00), (0, 2, 1, 0x3800), (1, 7, 0, 0x3400), (1, 1, 1, 0x3000)]


# ------------------------------------------------------------------------ wave planner
# tests/Shrike/Core/Kernels/Prefill/PrefillGroupedRoutedMoETests+Execution.swift

RANGES = [(0, 0, 40), (1, 40, 32), (2, 72, 5), (3, 77, 3)]


def blk(slot, ps, rows, staging, tile=None):
    return (slot, ps, rows, staging, staging // 64 if tile is None else tile)


def test_wave_planner_splits_and_pads():  # :382-432
    one = H.plan_expert_waves(RANGES, [0, 1, 2, 3], 512)
    assert one == [H.Wave([blk(0, 0, 40, 0), blk(1, 40, 32, 64), blk(2, 72, 5, 128), blk(3, 77, 3, 192)], 256)]
    assert H.row_tile_table(one[0]) == [0, 1, 2, 3]
    two = H.plan_expert_waves(RANGES, [0, 1, 2, 3], 128)
    assert two == [H.Wave([blk(0, 0, 40, 0), blk(1, 40, 32, 64)], 128), H.Wave([blk(2, 72, 5, 0), blk(3, 77, 3, 64)], 128)]
    long = H.plan_expert_waves([(2, 0, 600)], [0, 1, 2, 3], 512)
    assert long == [H.Wave([blk(2, 0, 512, 0)], 512), H.Wave([blk(2, 512, 88, 0)], 128)]
    assert len(H.row_tile_table(long[0])) == 8 and H.row_tile_table(long[1]) == [0, 0]
    with pytest.raises(H.PlanError):
        H.plan_expert_waves(RANGES, [0, 1, 2, 3], 96)


def test_tail_tile_planner():  # :535-577
    waves = H.plan_expert_waves(RANGES, [0, 1, 2, 3], 512, tail_tile=32)
    assert waves == [H.Wave([blk(0, 0, 40, 0, 0), blk(1, 40, 32, 64, 0), blk(2, 72, 5, 96, 1), blk(3, 77, 3, 128, 2)], 160, 96)]
    assert H.row_tile_tables(waves[0]) == ([0, 0, 1, 2, 3], [0], [1, 2, 3])
    split = H.plan_expert_waves(RANGES, [0, 1, 2, 3], 64, tail_tile=32)
    assert split == [H.Wave([blk(0, 0, 40, 0, 0)], 64, 0),
                     H.Wave([blk(1, 40, 32, 0, 0), blk(2, 72, 5, 32, 1)], 64, 64),
                     H.Wave([blk(3, 77, 3, 0, 0)], 32, 32)]
    long = H.plan_expert_waves([(2, 0, 200)], [0, 1, 2, 3], 128, tail_tile=32)
    assert long == [H.Wave([blk(2, 0, 128, 0, 0)], 128, 0), H.Wave([blk(2, 128, 64, 0, 0), blk(2, 192, 8, 64, 0)], 96, 32)]


def test_tail_tile_skipped_without_remainders():  # :603-622
    waves = H.plan_expert_waves([(0, 0, 64), (1, 64, 128), (2, 192, 97)], [0, 1, 2], 512, tail_tile=32)
    assert len(waves) == 1 and waves[0].tail_rows == 0 and waves[0].padded_rows == 320
    assert [b[2] for b in waves[0].blocks] == [64, 128, 97]
    assert [b[3] for b in waves[0].blocks] == [0, 64, 192]
    g, b, t = H.row_tile_tables(waves[0])
    assert t == [] and b == [0, 1, 1, 2, 2] and g == [0, 0, 1, 1, 1, 1, 2, 2, 2, 2]


def test_thirty_two_row_planner():  # :637-655
    waves = H.plan_expert_waves(RANGES, [0, 1, 2, 3], 512, row_tile=32)
    assert len(waves) == 1 and waves[0].padded_rows == 160
    assert [b[3] for b in waves[0].blocks] == [0, 64, 96, 128]
    assert [b[4] for b in waves[0].blocks] == [0, 2, 3, 4]
    assert H.row_tile_table(waves[0], 32) == [0, 0, 1, 2, 3]


def test_single_one_pair_expert():  # :736-739
    g = H.group_token_expert_pairs([P(0, 5, 0, 0)], 1, 1, 8, 16)
    ranges = [(e, s, c) for e, s, c in g.groups]
    assert H.plan_expert_waves(ranges, [5], 64) == [H.Wave([(0, 0, 1, 0, 0)], 64)]


# --------------------------------------------------------------------------- slot pool
# tests/Shrike/Core/Infrastructure/Streaming/PreadExpertStreamerTests+CachePlanning.swift, +Reading.swift

def test_planned_load_executes_same_misses():  # +CachePlanning:24-44
    c = H.SlotCache(4, 8)
    c.load([0])
    plan = c.plan([0, 1, 2])
    assert plan.hits == 1 and [plan.experts[i] for i in plan.misses] == [1, 2]


def test_resident_snapshot_excludes_loading():  # :46-62
    c = H.SlotCache(4, 8)
    c.load([1, 3])
    assert c.resident_experts() == [1, 3]
    plan = c.plan([2])
    assert plan.misses == [0] and c.resident_experts() == [1, 3]
    c.complete(plan)
    assert c.resident_experts() == [1, 2, 3]


def test_avoiding_slots():  # :130-154
    c = H.SlotCache(4, 8)
    c.load([0, 1])
    plan = c.plan([0, 2], avoiding_slots={0, 1})
    assert plan.assigned_slots == [0, 2] and plan.hits == 1 and plan.misses == [1]


def test_unplaceable_returns_none():  # :156-169
    c = H.SlotCache(4, 8)
    c.load([0, 1])
    assert c.plan([0, 2, 3, 4], avoiding_slots={0, 1}) is None


def _protecting(experts, n=8):
    return [e in experts for e in range(n)]


def test_protected_experts():  # :171-223
    def warmed():
        c = H.SlotCache(2, 8)
        c.load([0]); c.load([1]); c.load([0])
        return c
    p = warmed().plan([2])
    assert p.misses == [0] and p.assigned_slots == [1]
    p = warmed().plan([2], protected_experts=_protecting([1]))
    assert p.misses == [0] and p.assigned_slots == [0]
    c = H.SlotCache(2, 8)
    c.load([0, 1])
    assert c.plan([2], protected_experts=_protecting([0])).assigned_slots == [1]
    c = H.SlotCache(2, 8)
    c.load([0, 1])
    p = c.plan([2], protected_experts=_protecting([0, 1]))
    assert p.misses == [0] and p.assigned_slots[0] in (0, 1)


def test_pins_block_eviction():  # :225-244
    c = H.SlotCache(2, 8)
    c.load([0, 1])
    resident = c.plan([0, 1])
    c.pin(resident)
    assert c.counts()["pinned"] == 2
    assert c.plan([2]) is None
    c.unpin(resident.assigned_slots, resident.assigned_generations)
    assert c.counts()["pinned"] == 0
    c.complete(c.plan([2]))
    assert c.counts()["resident"] == 2


def test_statistics():  # :246-270
    c = H.SlotCache(2, 8)
    c.load([0, 1]); c.load([0, 2]); c.load([0, 1])
    s = c.stats
    assert (s["plans"], s["requested"], s["hits"], s["misses"]) == (3, 6, 2, 4)
    assert (s["read_operations"], s["evictions"], s["reloads"], s["load_batches"]) == (4, 2, 1, 3)
    assert c.counts()["loading"] == 0


def test_abandon_releases_slots():  # :320-341
    c = H.SlotCache(2, 8)
    c.load([0, 1])
    dropped = c.plan([2, 3])
    assert len(dropped.misses) == 2 and c.counts()["loading"] == 2
    assert c.plan([0]) is None
    c.abandon(dropped)
    assert c.counts()["loading"] == 0
    p = c.load([0, 1])
    assert sorted(p.assigned_slots) == [0, 1]


def test_slot_reuse_order():  # +Reading:26-53: experts 0,1,2,3 land in slots 0,1,0,1
    c = H.SlotCache(2, 8)
    slots = [c.load([e]).assigned_slots[0] for e in range(4)]
    assert slots == [0, 1, 0, 1]


def test_residency_words_follow_the_states():
    c = H.SlotCache(2, 4, first_cell=6)
    p = c.plan([3])
    assert c.words[3] == (H.LOADING << 32) | 6
    c.complete(p)
    assert c.words[3] == (H.RESIDENT << 32) | 6
    c.load([1]); c.load([2])  # evicts expert 3 (least used, oldest)
    assert c.words[3] == (H.EMPTY << 32) | U
    assert c.words[2] == (H.RESIDENT << 32) | 6
