"""The routed-tile loop of a streamed prefill chunk: the library's scheduler, sequencer, chunk protection and
slot-lifetime guard against the oracle's restatement and the vectors of the reference's own tests
(tests/Shrike/Core/Kernels/Prefill/PrefillRoutedTileSchedulerTests.swift, PrefillRoutedTileSequencerTests.swift)."""
import pytest

from oracle import host_logic as HL
from shrike_amd import host as H

DECISION = {H.ISSUE_WITHOUT_PENDING: ("issueWithoutPending", None),
            H.DRAIN_NO_ASSIGNED_SLOTS: ("drainBeforeIssue", "pendingTileHasNoAssignedSlots"),
            H.DRAIN_PLAN_UNAVAILABLE: ("drainBeforeIssue", "avoidingSlotPlanUnavailable"),
            H.DRAIN_MAX_DEPTH: ("drainBeforeIssue", "maxPendingDepthReached")}
CLOSE = {H.BATCH_OPEN: None, H.BATCH_FULL: "batchFull", H.BATCH_LAST_TILE: "lastTile"}


def both_configs(**kw):
    return H.TileSchedulerConfig(**kw), HL.TileConfig(**kw)


def decide(kw, has_pending, slots, available, depth=None):
    lib_cfg, ref_cfg = both_configs(**kw)
    code = H.TileScheduler(lib_cfg).decide(has_pending, slots, available, depth)
    got = ("prefetchNext", list(slots)) if code == H.PREFETCH_NEXT else DECISION[code]
    assert got == HL.tile_decide(ref_cfg, has_pending, slots, available, depth)
    return got


def batch_action(kw, tiles, slots, available, last):
    lib_cfg, ref_cfg = both_configs(**kw)
    before, after = H.TileScheduler(lib_cfg).batch_action(tiles, slots, available, last)
    got = (before, CLOSE[after])
    assert got == HL.tile_batch_action(ref_cfg, tiles, slots, available, last)
    return got


def fitting(kw, slot_count, reserved=0):
    lib_cfg, ref_cfg = both_configs(**kw)
    got, ref = lib_cfg.fitting(slot_count, reserved), ref_cfg.fitting(slot_count, reserved)
    assert (got.astuple() if got else None) == (ref.astuple() if ref else None)
    assert lib_cfg.fits_slot_budget(slot_count, reserved) == ref_cfg.fits_slot_budget(slot_count, reserved)
    return got.astuple() if got else None


# ------------------------------------------------------------------ scheduler (PrefillRoutedTileSchedulerTests.swift)

def test_decisions():
    assert decide({}, False, [], False) == ("issueWithoutPending", None)                                    # :7-14
    assert decide({}, True, [3, 7, 8], True) == ("prefetchNext", [3, 7, 8])                                 # :16-23
    assert decide({}, True, [], True) == ("drainBeforeIssue", "pendingTileHasNoAssignedSlots")              # :25-32
    assert decide({}, True, [1, 2], False) == ("drainBeforeIssue", "avoidingSlotPlanUnavailable")           # :34-41
    deep = dict(max_pending_depth=2, tile_experts=4)
    assert decide(deep, True, [1, 2, 3, 4, 5, 6, 7, 8], True, 2) == ("prefetchNext", [1, 2, 3, 4, 5, 6, 7, 8])  # :43-54
    assert decide(deep, True, [1, 2], True, 3) == ("drainBeforeIssue", "maxPendingDepthReached")            # :56-65
    assert decide({}, True, [9, 1, 9, 3], True) == ("prefetchNext", [9, 1, 9, 3])                           # :91-99
    assert decide({}, True, [1, 2], True, 2) == ("drainBeforeIssue", "maxPendingDepthReached")              # :110-114
    three = dict(max_pending_depth=3, tile_experts=4)                                                        # :291-307
    assert decide(three, True, [1, 2, 3, 4], True, 3)[0] == "prefetchNext"
    assert decide(three, True, [1, 2, 3, 4], True, 4) == ("drainBeforeIssue", "maxPendingDepthReached")
    for kw in ({}, dict(tiles_per_command_buffer=1)):                                                        # :101-152
        assert decide(kw, True, [], True) == ("drainBeforeIssue", "pendingTileHasNoAssignedSlots")


def test_slot_budget_and_fitting():
    assert H.TileSchedulerConfig().fits_slot_budget(16)                                                      # :67-75
    assert H.TileSchedulerConfig(max_pending_depth=2, tile_experts=4).fits_slot_budget(16)
    assert not H.TileSchedulerConfig(max_pending_depth=2, tile_experts=8).fits_slot_budget(16)
    assert fitting({}, 8) == (1, 4, 1, 0) and fitting({}, 1) is None                                         # :77-89
    assert H.TileSchedulerConfig().fitting(8).fits_slot_budget(8)
    wide = dict(max_pending_depth=1, tile_experts=8, tiles_per_command_buffer=4)                             # :232-262
    assert H.TileSchedulerConfig(**wide).fits_slot_budget(64) and not H.TileSchedulerConfig(**wide).fits_slot_budget(32)
    assert fitting(wide, 64) == (1, 8, 4, 0)
    assert fitting(wide, 32) == (1, 8, 2, 0) and fitting(wide, 8) == (1, 4, 1, 0) and fitting(wide, 1) is None
    assert fitting({}, 16) == (1, 8, 1, 0)
    deep = dict(max_pending_depth=2)                                                                         # :264-273
    assert fitting(deep, 128) == (2, 8, 1, 0) and fitting(deep, 16) == (2, 5, 1, 0)
    assert fitting(deep, 8) == (2, 2, 1, 0) and fitting(deep, 2) is None
    assert H.TileSchedulerConfig(max_pending_depth=15).fits_slot_budget(128)                                 # :275-281
    assert not H.TileSchedulerConfig(max_pending_depth=16).fits_slot_budget(128)
    look = dict(max_pending_depth=2, tile_experts=8, fetch_lookahead=1)                                      # :404-414
    assert H.TileSchedulerConfig(**look).fits_slot_budget(128) and not H.TileSchedulerConfig(**look).fits_slot_budget(31)
    assert H.TileSchedulerConfig(max_pending_depth=14, tile_experts=8, fetch_lookahead=1).fits_slot_budget(128)
    assert not H.TileSchedulerConfig(max_pending_depth=15, tile_experts=8, fetch_lookahead=1).fits_slot_budget(128)
    look = dict(max_pending_depth=2, fetch_lookahead=1)                                                      # :416-425
    assert fitting(look, 128) == (2, 8, 1, 1) and fitting(look, 16) == (2, 4, 1, 1)
    assert fitting(look, 8) == (2, 2, 1, 1) and fitting(look, 3) is None
    for slots in range(0, 140):
        for reserved in (0, 3):
            for kw in ({}, wide, deep, look, dict(max_pending_depth=4, tile_experts=3, tiles_per_command_buffer=7, fetch_lookahead=1)):
                fitting(kw, slots, reserved)


def test_config_clamps():
    assert H.TileSchedulerConfig(tiles_per_command_buffer=0).astuple()[2] == 1                               # :224-229
    assert H.TileSchedulerConfig(tiles_per_command_buffer=99).astuple()[2] == 16
    assert H.TileSchedulerConfig(max_pending_depth=0).astuple()[0] == 1                                      # :283-285
    assert H.TileSchedulerConfig(tile_experts=40, fetch_lookahead=5).astuple() == (1, 16, 1, 1)
    assert H.TileSchedulerConfig(tile_experts=0, fetch_lookahead=-2).astuple() == HL.TileConfig(tile_experts=0, fetch_lookahead=-2).astuple()


def test_batch_actions():
    one = dict(tiles_per_command_buffer=1)                                                                   # :136-151
    assert batch_action(one, 0, [], True, False) == (False, "batchFull")
    assert batch_action(one, 0, [], True, True) == (False, "batchFull")
    four = dict(tiles_per_command_buffer=4)
    assert batch_action(four, 2, [1, 2], True, False) == (False, None)                                       # :154-169
    assert batch_action(four, 3, [1, 2], True, False) == (False, "batchFull")
    assert batch_action(four, 2, [2, 5], False, False) == (True, None)                                       # :171-186
    assert batch_action(four, 2, [], False, False) == (False, None)
    assert batch_action(four, 1, [2, 5], True, True) == (False, "lastTile")                                  # :188-203
    assert batch_action(four, 0, [], True, True) == (False, "lastTile")
    assert batch_action(four, 3, [2, 5], True, True) == (False, "batchFull")                                 # :205-214
    assert batch_action(four, 2, [2, 5], False, True) == (True, "lastTile")                                  # :216-222
    assert batch_action({}, 1, [2, 5], False, False) == (True, "batchFull")


def test_lookahead_needs_a_lookahead_a_plan_and_a_successor():                                               # :427-440
    with_, without = H.TileScheduler(H.TileSchedulerConfig(fetch_lookahead=1)), H.TileScheduler()
    assert with_.should_begin_lookahead(0, 3, True)
    assert not without.should_begin_lookahead(0, 3, True)
    assert not with_.should_begin_lookahead(0, 3, False)
    assert not with_.should_begin_lookahead(2, 3, True)
    assert with_.plans_lookahead(1, 3) and not with_.plans_lookahead(2, 3)


def test_chunk_expert_protection():                                                                          # :336-370
    p = H.ChunkExpertProtection([1, 2, 3, 4, 5], 10)
    assert p.remaining == [False, True, True, True, True, True, False, False, False, False]
    p.planning([1, 2])
    assert p.remaining == [False, False, False, True, True, True, False, False, False, False]
    p.planning([3])
    assert p.remaining == [False, False, False, False, True, True, False, False, False, False]
    p.planning([4, 5])
    assert not any(p.remaining)
    p = H.ChunkExpertProtection([1, 2], 10)
    p.planning([9, -1, 40])
    assert p.remaining[1] and p.remaining[2] and not p.remaining[9]
    assert H.ChunkExpertProtection([2, 7, 12, -3], 10).remaining == [False, False, True, False, False, False, False, True, False, False]


def test_slot_lifetime():                                                                                    # :372-402
    life = H.TileSlotLifetime()
    life.begin(0, [1, 2])
    with pytest.raises(H.TileLifetimeError) as e:
        life.begin(1, [2, 3])
    assert e.value.code == 2 and e.value.conflicting_tile == 0
    life.complete(0)
    life.begin(1, [2, 3])
    life = H.TileSlotLifetime()
    life.begin(0, [1, 2])
    life.begin(1, [3, 4])
    with pytest.raises(H.TileLifetimeError):
        life.begin(2, [2, 4])
    life.complete(0)
    with pytest.raises(H.TileLifetimeError) as e:
        life.begin(2, [4, 5])
    assert e.value.conflicting_tile == 1
    life.complete(1)
    life.begin(2, [4, 5])
    with pytest.raises(H.TileLifetimeError) as e:
        life.begin(3, [7, 7])
    assert e.value.code == 1
    with pytest.raises(H.TileLifetimeError) as e:
        life.complete(9)
    assert e.value.code == 3


# ------------------------------------------------------------------ sequencer (PrefillRoutedTileSequencerTests.swift)

class EncodeFailure(Exception):
    pass


class BeginFailure(Exception):
    pass


class RecordingDriver:
    """PrefillRoutedTileSequencerTests.RecordingDriver (:24-105): records only a commit that seals a non-empty batch."""

    def __init__(self):
        self.calls, self.plan_refusals, self.failing_encodes, self.failing_begins = [], {}, set(), set()
        self.slots_per_tile = 2
        self.open_tiles, self.pending = [], []
        self.kept, self.begun, self.abandoned_begun, self.abandoned_kept = set(), set(), set(), set()

    def _slots(self, tile):
        return [tile * self.slots_per_tile + i for i in range(self.slots_per_tile)]

    open_batch_tiles = property(lambda self: len(self.open_tiles))
    open_batch_slots = property(lambda self: [s for t in self.open_tiles for s in self._slots(t)])
    pending_depth = property(lambda self: len(self.pending))
    pending_assigned_slots = property(lambda self: [s for b in self.pending for s in b])

    def plan(self, tile, avoiding_in_flight):
        self.calls.append(("plan", tile, avoiding_in_flight))
        if self.plan_refusals.get(tile, 0) > 0:
            self.plan_refusals[tile] -= 1
            return False
        self.kept.add(tile)
        return True

    def begin(self, tile):
        self.calls.append(("begin", tile))
        self.kept.discard(tile)
        if tile in self.failing_begins:
            raise BeginFailure(tile)
        self.begun.add(tile)

    def abandon_plan(self, tile):
        self.calls.append(("abandonPlan", tile))
        self.kept.discard(tile)

    def encode(self, tile):
        self.calls.append(("encode", tile))
        if tile in self.failing_encodes:
            raise EncodeFailure(tile)
        self.begun.discard(tile)
        self.open_tiles.append(tile)

    def commit_open_batch(self):
        if not self.open_tiles:
            return
        self.calls.append("commit")
        self.pending.append(self.open_batch_slots)
        self.open_tiles = []

    def drain_oldest_batch(self):
        self.calls.append("drain")
        if self.pending:
            self.pending.pop(0)

    def abandon_begun_fetches(self):
        self.calls.append("abandonBegun")
        self.abandoned_begun, self.abandoned_kept = set(self.begun), set(self.kept)
        self.begun, self.kept = set(), set()


def P(tile, avoiding=None):
    return ("plan", tile, avoiding)


def B(tile):
    return ("begin", tile)


def E(tile):
    return ("encode", tile)


CASES = {
    # name: (setup, tiles, depth, width, lookahead, expected calls)
    "lookahead begins the successor before the tile is awaited": (
        {}, 3, 2, 1, 1,
        [P(0), B(0), P(1, 0), B(1), E(0), "commit", P(2, 1), B(2), E(1), "commit", E(2), "commit", "drain", "drain", "drain"]),
    "without a lookahead each tile is begun at its own turn": (
        {}, 3, 2, 1, 0,
        [P(0), B(0), E(0), "commit", P(1), B(1), E(1), "commit", P(2), B(2), E(2), "commit", "drain", "drain", "drain"]),
    "a single tile begins no successor": ({}, 1, 2, 1, 1, [P(0), B(0), E(0), "commit", "drain"]),
    "no tiles, no calls": ({}, 0, 2, 1, 1, []),
    "an unplaceable tile commits the open batch and drains it before replanning": (
        dict(plan_refusals={1: 1}), 2, 2, 2, 0,
        [P(0), B(0), E(0), P(1), "commit", "drain", B(1), E(1), "commit", "drain"]),
    "the valve holds at the lookahead depth too": (
        dict(plan_refusals={1: 2}), 2, 2, 2, 1,
        [P(0), B(0), P(1, 0), E(0), P(1), "commit", "drain", B(1), E(1), "commit", "drain"]),
    "a declined lookahead is planned again at its own turn": (
        dict(plan_refusals={1: 1}), 2, 2, 1, 1,
        [P(0), B(0), P(1, 0), E(0), "commit", P(1), B(1), E(1), "commit", "drain", "drain"]),
    "the open batch counts against the depth with the committed ones": (
        {}, 3, 1, 2, 0,
        [P(0), B(0), E(0), P(1), B(1), E(1), "commit", P(2), B(2), E(2), "commit", "drain", "drain"]),
    "a pending batch without slots is drained and the kept plan abandoned": (
        dict(slots_per_tile=0), 2, 2, 1, 0,
        [P(0), B(0), E(0), "commit", P(1), ("abandonPlan", 1), "drain", B(1), E(1), "commit", "drain"]),
}


def run_both(setup, tiles, depth, width, lookahead):
    out = []
    kw = dict(max_pending_depth=depth, tiles_per_command_buffer=width, fetch_lookahead=lookahead)
    for runner in ("library", "oracle"):
        driver = RecordingDriver()
        for k, v in setup.items():
            setattr(driver, k, dict(v) if isinstance(v, dict) else set(v) if isinstance(v, set) else v)
        error = None
        try:
            if runner == "library":
                H.TileSequencer(H.TileScheduler(H.TileSchedulerConfig(**kw))).run(tiles, driver)
            else:
                HL.tile_sequence(HL.TileConfig(**kw), tiles, driver)
        except (EncodeFailure, BeginFailure) as exc:
            error = exc
        out.append((driver, error))
    assert out[0][0].calls == out[1][0].calls, "library and oracle drive the driver differently"
    assert type(out[0][1]) is type(out[1][1])
    return out[0]


@pytest.mark.parametrize("name", list(CASES))
def test_sequencer_traces(name):
    setup, tiles, depth, width, lookahead, expected = CASES[name]
    driver, error = run_both(setup, tiles, depth, width, lookahead)
    assert error is None
    assert driver.calls == expected


def test_a_failure_waits_out_every_begun_fetch_and_propagates():                                             # :219-239
    driver, error = run_both(dict(failing_encodes={0}), 3, 2, 1, 1)
    assert isinstance(error, EncodeFailure) and error.args == (0,)
    assert driver.calls == [P(0), B(0), P(1, 0), B(1), E(0), "abandonBegun"]
    assert driver.abandoned_begun == {0, 1} and not driver.abandoned_kept and not driver.begun and not driver.kept


def test_a_failure_inside_a_begin_still_waits_out_the_begun_predecessor():                                   # :241-261
    driver, error = run_both(dict(failing_begins={1}), 3, 2, 1, 1)
    assert isinstance(error, BeginFailure) and error.args == (1,)
    assert driver.calls == [P(0), B(0), P(1, 0), B(1), "abandonBegun"]
    assert driver.abandoned_begun == {0} and not driver.abandoned_kept and not driver.begun and not driver.kept


def test_sequencer_random_drivers_agree_with_the_oracle():
    import random
    rng = random.Random(11)
    for _ in range(200):
        tiles = rng.randint(0, 9)
        setup = dict(plan_refusals={t: rng.randint(0, 2) for t in range(tiles) if rng.random() < 0.3},
                     slots_per_tile=rng.choice([0, 1, 2, 3]))
        if rng.random() < 0.2 and tiles:
            setup["failing_encodes"] = {rng.randrange(tiles)}
        if rng.random() < 0.2 and tiles:
            setup["failing_begins"] = {rng.randrange(tiles)}
        run_both(setup, tiles, rng.randint(1, 4), rng.randint(1, 4), rng.randint(0, 1))
