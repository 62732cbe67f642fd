"""The predictive prefetch ring and its load operations: the library and the oracle's restatement against
every case of the reference's tests/Shrike/Core/Runtime/ExpertPrefetchRingTests.swift."""
import threading
import time

import pytest

from oracle import host_logic as HL
from shrike_amd import host as H


class Library:
    Operation, Refused = H.ExpertLoadOperation, H.PrefetchClaimRefused

    @staticmethod
    def ring(cells, drop):
        return H.ExpertPrefetchRing(cells, drop)

    @staticmethod
    def fail(op):
        op.finish(5)


class Oracle:
    Operation, Refused = HL.LoadOperation, HL.ClaimRefused

    @staticmethod
    def ring(cells, drop):
        return HL.PrefetchRing(cells, drop)

    @staticmethod
    def fail(op):
        op.finish("read failed")


@pytest.fixture(params=[Library, Oracle], ids=["library", "oracle"])
def impl(request):
    return request.param


def make(impl, cells=(10, 11, 12, 13)):
    drops = []
    return impl.ring(list(cells), lambda layer, expert, cell: drops.append((layer, expert, cell))), drops


def later(seconds, fn):
    t = threading.Timer(seconds, fn)
    t.start()
    return t


def test_begin_keeps_the_in_flight_budget_and_frees_it_when_a_read_completes(impl):          # :24-56
    ring, _ = make(impl)
    issued, first, second = [], impl.Operation(), impl.Operation()

    def issue_first(experts, cells):
        issued.append(experts)
        assert len(cells) == len(experts) and all(10 <= c <= 13 for c in cells)
        return first

    ring.begin(3, [7, 9, 11], [], issue=issue_first)
    assert issued == [[7]] and ring.in_flight_count == 1

    def issue_second(experts, cells):
        issued.append(experts)
        return second

    ring.begin(4, [1, 2], [], issue=issue_second)
    assert issued == [[7]] and ring.statistics["issued"] == 1
    first.mark_in_flight()
    first.finish()
    ring.begin(4, [1, 2], [], issue=issue_second)
    assert issued == [[7], [1]]
    assert ring.statistics["issued"] == 2 and ring.statistics["reclaimed"] == 1


def test_begin_dedupes_resident_and_active_predictions(impl):                                # :58-73
    ring, _ = make(impl)
    issued, first = [], impl.Operation()
    ring.begin(2, [1, 2, 3], [2], issue=lambda e, c: (issued.append(e), first)[1])
    first.finish()
    ring.begin(2, [1, 3, 4, 4], [], issue=lambda e, c: (issued.append(e), impl.Operation())[1])
    assert issued == [[1], [3]]
    assert ring.statistics["refused"] == 2


def test_ready_cells_waits_for_an_in_flight_prediction_and_counts_a_late_one(impl):          # :75-87
    ring, _ = make(impl)
    op = impl.Operation()
    ring.begin(2, [1], [], issue=lambda e, c: op)
    op.mark_in_flight()
    t = later(0.020, op.finish)
    ready = ring.ready_cells(2, [1, 5], join_nanos=1_000_000)
    t.join()
    assert ready == {1: 10}
    assert ring.statistics["late"] == 1 and ring.statistics["joined"] == 0


def test_ready_cells_joins_a_prediction_that_finishes_within_the_bound(impl):                # :89-101
    ring, _ = make(impl)
    op = impl.Operation()
    ring.begin(2, [1], [], issue=lambda e, c: op)
    op.mark_in_flight()
    t = later(0.002, op.finish)
    ready = ring.ready_cells(2, [1, 2], join_nanos=500_000_000)
    t.join()
    assert ready == {1: 10}
    assert ring.statistics["joined"] == 1 and ring.statistics["late"] == 0


def test_ready_cells_skips_a_failed_prediction_and_a_claimed_slot_awaiting_its_attach(impl):  # :103-119
    ring, _ = make(impl)
    failed = impl.Operation()
    ring.begin(2, [1], [], issue=lambda e, c: failed)
    failed.mark_in_flight()
    impl.fail(failed)
    assert ring.ready_cells(2, [1], join_nanos=1_000_000) == {}
    assert ring.statistics["late"] == 0
    seen = {}

    def issue(experts, cells):
        assert ring.ready_cells(3, [4], join_nanos=1_000_000) == {}
        seen["late"] = ring.statistics["late"]
        return impl.Operation()

    ring.begin(3, [4], [], issue=issue)
    assert seen["late"] == 1


def test_consume_moves_the_entry_to_the_cell_the_pool_freed(impl):                           # :121-136
    ring, _ = make(impl)
    op = impl.Operation()
    ring.begin(2, [1], [], issue=lambda e, c: op)
    op.finish()
    assert ring.ready_cells(2, [1]) == {1: 10}
    ring.consume(2, {1}, {1: 77})
    assert ring.statistics["adopted"] == 1
    cells_seen = []
    ring.begin(3, [5], [], issue=lambda e, c: (cells_seen.extend(c), impl.Operation())[1])
    assert cells_seen == [77]


def test_consume_without_a_freed_cell_keeps_the_rings_cell_and_drops_the_landing(impl):      # :138-166
    ring, drops = make(impl)
    op = impl.Operation()
    ring.begin(2, [1], [], issue=lambda e, c: op)
    op.finish()
    ring.ready_cells(2, [1])
    ring.consume(2, {1}, {})
    assert drops == [(2, 1, 10)]
    cells_seen = []
    ring.begin(3, [5], [], issue=lambda e, c: (cells_seen.extend(c), impl.Operation())[1])
    assert cells_seen == [10]


def test_a_refused_claim_is_counted_and_its_slots_freed(impl):                               # :168-184
    ring, _ = make(impl)

    def refuse(experts, cells):
        raise impl.Refused()

    ring.begin(2, [1, 2], [], issue=refuse)
    st = ring.statistics
    assert st["refused"] == 2 and st["issued"] == 0 and st["hook_failures"] == 0 and ring.in_flight_count == 0
    issued = []
    ring.begin(2, [1, 2], [], issue=lambda e, c: (issued.append(e), impl.Operation())[1])
    assert issued == [[1]]


def test_the_reclaim_keeps_the_layer_whose_plan_is_still_to_come(impl):                      # :186-201
    ring, drops = make(impl)
    past, pending = impl.Operation(), impl.Operation()
    ring.begin(1, [1], [], issue=lambda e, c: past)
    past.finish()
    ring.begin(3, [3], [], issue=lambda e, c: pending)
    pending.finish()
    ring.begin(3, [4], [], issue=lambda e, c: impl.Operation())
    assert len(drops) == 1 and drops[0][0] == 1
    assert ring.statistics["reclaimed"] == 1
    assert ring.ready_cells(3, [3]) == {3: 10}


def test_a_leased_slot_is_never_reclaimed_by_another_layers_begin(impl):                     # :203-232
    ring, drops = make(impl)
    op = impl.Operation()
    ring.begin(2, [1], [], issue=lambda e, c: op)
    op.finish()
    leased = ring.ready_cells(2, [1])[1]
    cells_seen, nxt = [], impl.Operation()
    ring.begin(3, [5], [], issue=lambda e, c: (cells_seen.extend(c), nxt)[1])
    assert cells_seen == [11] and leased not in cells_seen
    assert ring.statistics["reclaimed"] == 0 and drops == []
    ring.consume(2, {1}, {1: 40})
    nxt.finish()
    cells_seen.clear()
    ring.begin(4, [8], [], issue=lambda e, c: (cells_seen.extend(c), impl.Operation())[1])
    assert cells_seen == [40]


def test_the_reclaim_drops_a_completed_landing_before_its_cell_is_reused(impl):              # :234-251
    ring, drops = make(impl, cells=[10])
    op = impl.Operation()
    ring.begin(2, [1], [], issue=lambda e, c: op)
    op.finish()
    cells_seen = []

    def issue(experts, cells):
        cells_seen.extend(cells)
        assert len(drops) == 1
        return impl.Operation()

    ring.begin(3, [5], [], issue=issue)
    assert cells_seen == [10] and ring.statistics["reclaimed"] == 1 and drops == [(2, 1, 10)]


def test_the_reclaim_of_a_failed_prediction_drops_nothing(impl):                             # :253-266
    ring, drops = make(impl, cells=[10])
    op = impl.Operation()
    ring.begin(2, [1], [], issue=lambda e, c: op)
    op.mark_in_flight()
    impl.fail(op)
    ring.begin(3, [5], [], issue=lambda e, c: impl.Operation())
    st = ring.statistics
    assert drops == [] and st["reclaimed"] == 0 and st["failed"] == 1 and st["issued"] == 2


def test_unlease_returns_a_throwing_plans_predictions_to_the_ring(impl):                     # :268-287
    ring, drops = make(impl)
    op = impl.Operation()
    ring.begin(2, [1], [], issue=lambda e, c: op)
    op.finish()
    leased = ring.ready_cells(2, [1])[1]
    ring.unlease(2, {1})
    cells_seen = []
    ring.begin(3, [5], [], issue=lambda e, c: (cells_seen.extend(c), impl.Operation())[1])
    st = ring.statistics
    assert cells_seen == [leased] and st["reclaimed"] == 1 and st["adopted"] == 0 and len(drops) == 1


def test_demand_submissions_count_the_reads_they_overlap(impl):                              # :289-300
    ring, _ = make(impl)
    ring.note_demand_submission()
    assert ring.statistics["overlapped"] == 0
    op = impl.Operation()
    ring.begin(2, [1], [], issue=lambda e, c: op)
    ring.note_demand_submission()
    assert ring.statistics["overlapped"] == 1
    op.finish()
    ring.note_demand_submission()
    assert ring.statistics["overlapped"] == 1


def test_begin_records_deferred_issues_and_their_wall(impl):                                 # :302-311
    ring, _ = make(impl)
    first = impl.Operation()
    ring.begin(2, [1], [], deferred=True, issue=lambda e, c: first)
    first.finish()
    ring.begin(3, [2], [], issue=lambda e, c: impl.Operation())
    st = ring.statistics
    assert st["deferred"] == 1 and st["issued"] == 2 and st["begin_nanos"] > 0


def test_completion_nanos_reports_completed_predictions_only(impl):                          # :313-331
    ring, _ = make(impl)
    first, second = impl.Operation(), impl.Operation()
    ring.begin(2, [1], [], issue=lambda e, c: first)
    before = time.monotonic_ns()
    first.finish()
    ring.begin(2, [5], [], issue=lambda e, c: second)
    stamps = ring.completion_nanos(2, [1, 5, 9])
    assert sorted(stamps) == [1] and stamps[1] >= before
    assert ring.completion_nanos(3, [1]) == {}
    impl.fail(second)
    assert ring.completion_nanos(2, [5]) == {}
    ring.consume(2, {1}, {})
    assert ring.completion_nanos(2, [1]) == {}


def test_predictions_beyond_the_budget_or_the_cells_are_counted_as_refused(impl):            # :333-340
    ring, _ = make(impl)
    ring.begin(2, [1, 2, 3], [], issue=lambda e, c: impl.Operation())
    assert ring.statistics["refused"] == 2
    ring.begin(3, [4], [], issue=lambda e, c: impl.Operation())
    assert ring.statistics["refused"] == 3 and ring.statistics["issued"] == 1


def test_the_first_hook_failure_is_the_one_to_log(impl):                                     # :342-347
    ring, _ = make(impl, cells=[10, 11])
    assert ring.note_hook_failure() and not ring.note_hook_failure()
    assert ring.statistics["hook_failures"] == 2


def test_begin_rolls_the_slots_back_when_the_issue_throws(impl):                             # :349-364
    class ReaderRefused(Exception):
        pass

    ring, _ = make(impl)

    def throw(experts, cells):
        raise ReaderRefused()

    with pytest.raises(ReaderRefused):
        ring.begin(2, [1, 2], [], issue=throw)
    assert ring.in_flight_count == 0 and ring.statistics["issued"] == 0
    issued = []
    ring.begin(2, [1, 2], [], issue=lambda e, c: (issued.append(e), impl.Operation())[1])
    assert issued == [[1]]


def test_claim_demand_leases_free_cells_outside_the_prediction_budget_and_consume_frees_them(impl):  # :366-393
    ring, drops = make(impl)
    prediction = impl.Operation()
    ring.begin(2, [1], [], issue=lambda e, c: prediction)
    prediction.mark_in_flight()
    claimed = ring.claim_demand(2, [7, 8])
    assert claimed == {7: 11, 8: 12} and ring.statistics["leased_peak"] == 2
    demand = impl.Operation()
    ring.attach_demand(2, set(claimed), demand)
    demand.mark_in_flight()
    demand.finish()
    assert ring.in_flight_count == 1
    ring.begin(3, [5], [], issue=lambda e, c: impl.Operation())
    assert drops == []
    ring.consume(2, set(claimed), {7: 20})
    assert [d[1] for d in drops] == [8]
    prediction.finish()
    again = ring.claim_demand(4, [9, 10, 11, 12, 13])
    assert [d[1] for d in drops] == [8, 1]
    assert set(again.values()) == {10, 20, 12, 13} and len(again) == 4


def test_claim_demand_reuses_the_layers_own_failed_slot(impl):                               # :395-403
    ring, _ = make(impl)
    failed = impl.Operation()
    ring.begin(2, [7], [], issue=lambda e, c: failed)
    failed.mark_in_flight()
    impl.fail(failed)
    assert ring.claim_demand(2, [7]) == {7: 10}
    assert ring.statistics["failed"] == 1


def test_claim_demand_never_doubles_a_prediction_still_in_flight(impl):                      # :405-407 ff.
    ring, _ = make(impl)
    op = impl.Operation()
    ring.begin(3, [9], [], issue=lambda e, c: op)
    op.mark_in_flight()
    assert ring.claim_demand(3, [9]) == {}
    assert ring.claim_demand(3, [4]) == {4: 11}


def test_geometry_and_operation_misuse(impl):
    with pytest.raises(Exception):
        impl.ring([], lambda *a: None)
    with pytest.raises(Exception):
        impl.ring([3, 3], lambda *a: None)
    op = impl.Operation()
    op.mark_in_flight()
    with pytest.raises(Exception):
        op.mark_in_flight()
    op.finish()
    with pytest.raises(Exception):
        op.finish()


def test_load_operation_waits_and_stamps():
    op = H.ExpertLoadOperation()
    assert op.state == H.LOAD_SUBMITTED and op.completed_nanos == 0
    assert not op.wait_until(H.monotonic_nanos() + 1_000_000)
    op.mark_in_flight()
    assert op.state == H.LOAD_IN_FLIGHT and op.started_nanos >= op.submitted_nanos
    t = later(0.005, lambda: op.finish(0))
    op.wait()
    t.join()
    assert op.state == H.LOAD_COMPLETED and op.completed_nanos >= op.started_nanos
    bad = H.ExpertLoadOperation()
    bad.finish(5)
    assert bad.state == H.LOAD_FAILED
    with pytest.raises(H.ReadFailed) as e:
        bad.wait()
    assert e.value.errno == 5
    assert bad.wait_until(0)


def test_two_threads_begin_and_plan_against_one_ring():
    """begin may run on a storage thread and on the decode thread at once (ExpertPrefetchRing.swift:38-41)."""
    drops = []
    ring = H.ExpertPrefetchRing([0, 1, 2, 3], lambda *a: drops.append(a))
    stop, errors = threading.Event(), []

    def storage():
        layer = 0
        try:
            while not stop.is_set():
                layer += 1
                op = H.ExpertLoadOperation()
                ring.begin(layer, [layer % 7, (layer + 1) % 7], [], issue=lambda e, c: op)
                if op.state == H.LOAD_SUBMITTED:
                    op.mark_in_flight()
                    op.finish(0 if layer % 5 else 5)
        except BaseException as exc:  # pragma: no cover
            errors.append(exc)

    t = threading.Thread(target=storage)
    t.start()
    try:
        for layer in range(1, 400):
            ready = ring.ready_cells(layer, list(range(7)), join_nanos=200_000)
            ring.consume(layer, set(ready), {})
            claimed = ring.claim_demand(layer, [8])
            ring.consume(layer, set(claimed), {})
    finally:
        stop.set()
        t.join()
    assert not errors
    st = ring.statistics
    assert st["issued"] > 0 and ring.leased_count == 0
