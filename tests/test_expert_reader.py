"""The parallel expert reader behind the reference's C interface, with the cases of the reference's own
tests (tests/Shrike/Core/Infrastructure/Streaming/ParallelExpertReaderTests.swift and
ParallelExpertReaderTests+BatchDepth.swift): whatever order the workers finish in, expert i lands in
destination i."""
import ctypes as C
import errno
import threading

import numpy as np
import pytest

from oracle import host_logic as HL
from shrike_amd import capi, host

STRIDE = 4096  # ParallelExpertReaderTests.swift:12


@pytest.fixture
def fixture_file(tmp_path):
    """Block e is filled with the byte e % 251 (ParallelExpertReaderTests.swift:16-25)."""
    def make(count):
        path = tmp_path / f"experts_{count}.bin"
        np.repeat((np.arange(count) % 251).astype(np.uint8), STRIDE).tofile(path)
        return str(path)
    return make


class Destinations:
    """n page-aligned buffers of one stride each."""

    def __init__(self, n):
        self.raw = np.zeros(n * STRIDE + 16384, np.uint8)
        base = self.raw.ctypes.data
        self.first = (base + 16383) // 16384 * 16384
        self.view = self.raw[self.first - base:self.first - base + n * STRIDE].reshape(n, STRIDE)
        self.view[:] = 0xEE
        self.addresses = [self.first + i * STRIDE for i in range(n)]


def test_reads_each_expert_into_its_own_destination(fixture_file):
    reader = host.ParallelExpertReader(fixture_file(64), STRIDE, threads=4)
    wanted = [63, 0, 17, 17, 40, 5, 62, 1]  # out of order, with a repeat
    dst = Destinations(len(wanted))
    reader.fetch(wanted, dst.addresses)
    for i, e in enumerate(wanted):
        assert dst.view[i, 0] == e % 251 and dst.view[i, -1] == e % 251, f"destination {i} wanted expert {e}"
        assert np.all(dst.view[i] == e % 251)


def test_single_threaded_matches_multi_threaded(fixture_file):
    path = fixture_file(32)
    ids = list(range(32))[::-1]
    firsts = []
    for threads in (1, 8):
        dst = Destinations(len(ids))
        host.ParallelExpertReader(path, STRIDE, threads=threads).fetch(ids, dst.addresses)
        firsts.append(dst.view[:, 0].copy())
    assert np.array_equal(firsts[0], firsts[1]) and np.array_equal(firsts[0], np.array(ids) % 251)


def test_repeated_batches_reuse_the_pool(fixture_file):
    reader = host.ParallelExpertReader(fixture_file(16), STRIDE, threads=4)
    dst = Destinations(4)
    for round_ in range(8):  # a lost wake-up between batches would hang here
        ids = [(round_ * 4 + i) % 16 for i in range(4)]
        reader.fetch(ids, dst.addresses)
        assert dst.view[:, 0].tolist() == [e % 251 for e in ids]


def _hammer(reader, ids_of_round, rounds, failures):
    try:
        dst = Destinations(4)
        for r in range(rounds):
            ids = ids_of_round(r)
            reader.fetch(ids, dst.addresses)
            if dst.view[:, 0].tolist() != [e % 251 for e in ids] or dst.view[:, -1].tolist() != [e % 251 for e in ids]:
                failures.append((r, ids, dst.view[:, 0].tolist()))
                return
    except Exception as exc:  # noqa: BLE001 - reported to the asserting thread
        failures.append(exc)


@pytest.mark.parametrize("depth", [1, 2])
def test_concurrent_callers_cannot_overwrite_a_published_batch(fixture_file, depth):
    """concurrentCallersCannotOverwritePublishedBatch and twoConcurrentFetchesBothLandTheirOwnBytes."""
    reader = host.ParallelExpertReader(fixture_file(64), STRIDE, threads=4, batch_depth=depth)
    failures = []
    workers = [threading.Thread(target=_hammer, args=(reader, (lambda r, w=w: [w * 32 + (r * 4 + i) % 32 for i in range(4)]),
                                                     50, failures)) for w in range(2)]
    [t.start() for t in workers]
    [t.join(60) for t in workers]
    assert not any(t.is_alive() for t in workers), "a fetch never returned"
    assert failures == []


def test_one_batchs_read_error_does_not_fail_the_other_caller(fixture_file):
    count = 16
    reader = host.ParallelExpertReader(fixture_file(count), STRIDE, threads=2, batch_depth=2)
    failures, errors = [], []

    def past_the_end():
        dst = Destinations(1)
        for _ in range(50):
            try:
                reader.fetch([count + 5], dst.addresses)
                errors.append("no error")
            except host.ReadFailed as exc:
                errors.append(exc.errno)

    good = threading.Thread(target=_hammer, args=(reader, lambda r: [(r * 4 + i) % count for i in range(4)], 50, failures))
    bad = threading.Thread(target=past_the_end)
    good.start(), bad.start()
    good.join(60), bad.join(60)
    assert not good.is_alive() and not bad.is_alive()
    assert failures == []
    assert errors == [errno.EIO] * 50  # a blob that runs past the end of the file (expert_io.c:113-115)


def test_depth_two_reads_the_same_bytes_as_depth_one(fixture_file):
    path = fixture_file(32)
    wanted = [31, 0, 15, 15, 20, 3, 30, 1]
    firsts = []
    for threads, depth in ((1, 1), (8, 2)):
        dst = Destinations(len(wanted))
        host.ParallelExpertReader(path, STRIDE, threads=threads, batch_depth=depth).fetch(wanted, dst.addresses)
        firsts.append(dst.view[:, 0].tolist())
    assert firsts[0] == firsts[1] == [e % 251 for e in wanted]


def test_fetch_by_absolute_offsets(fixture_file):
    reader = host.ParallelExpertReader(fixture_file(8), STRIDE, threads=3)
    dst = Destinations(3)
    reader.fetch_offsets([7 * STRIDE, 0, 3 * STRIDE + 512], dst.addresses)
    assert dst.view[0, 0] == 7 and dst.view[1, -1] == 0
    assert dst.view[2, 0] == 3 and dst.view[2, -1] == 4  # an offset inside block 3 runs into block 4


def test_empty_fetch_missing_file_end_of_file_and_clamping(fixture_file):
    path = fixture_file(4)
    reader = host.ParallelExpertReader(path, STRIDE)
    reader.fetch([], [])
    assert reader.thread_count >= 1
    with pytest.raises(host.ReadFailed) as e:
        host.ParallelExpertReader("/nonexistent/shrike/experts.bin", 4096)
    assert e.value.errno == errno.ENOENT
    with pytest.raises(host.ReadFailed) as e:
        host.ParallelExpertReader(fixture_file(2), STRIDE, threads=2).fetch([99], Destinations(1).addresses)
    assert e.value.errno == errno.EIO
    assert host.ParallelExpertReader(path, STRIDE, threads=0).thread_count == 1
    assert host.ParallelExpertReader(path, STRIDE, threads=999).thread_count == 16
    assert host.ParallelExpertReader(path, STRIDE, batch_depth=0).batch_depth == 1
    assert host.ParallelExpertReader(path, STRIDE, batch_depth=9).batch_depth == 2
    err = C.c_int(0)
    assert not capi.load().shrike_expert_reader_create(path.encode(), 0, 1, 1, 0, C.byref(err)) and err.value == errno.EINVAL
    assert capi.load().shrike_expert_reader_fetch(None, None, None, 1) == errno.EINVAL
    assert capi.load().shrike_expert_reader_threads(None) == 0


def test_bypassing_the_page_cache_reads_the_same_bytes_or_fails_at_open(fixture_file):
    """O_DIRECT where the file system has it; no silent fall-back where it has not (expert_io.c:216-229)."""
    path = fixture_file(16)
    try:
        reader = host.ParallelExpertReader(path, STRIDE, threads=2, bypass_cache=True)
    except host.ReadFailed as exc:
        assert exc.errno == errno.EINVAL  # this file system refuses O_DIRECT
        return
    dst = Destinations(4)
    reader.fetch([9, 2, 15, 0], dst.addresses)
    assert dst.view[:, 0].tolist() == [9, 2, 15, 0] and dst.view[:, -1].tolist() == [9, 2, 15, 0]


# ------------------------------------------------------------------ the pure rules

def _slots(rows):
    arr = (capi.ExpertBatchSlot * len(rows))()
    for i, (active, sequence, next_index, count) in enumerate(rows):
        arr[i] = capi.ExpertBatchSlot(active, sequence, next_index, count)
    return arr


@pytest.mark.parametrize("rows,claim", [  # claimTakesTheOlderBatchBeforeTheNewer (+BatchDepth.swift:56-80)
    ([(1, 5, 0, 2), (1, 6, 0, 2)], 0), ([(1, 5, 2, 2), (1, 6, 0, 2)], 1), ([(1, 5, 2, 2), (1, 6, 2, 2)], -1),
    ([(0, 1, 0, 2), (1, 6, 0, 2)], 1), ([(1, 9, 0, 1), (1, 3, 0, 1)], 1), ([], -1)])
def test_claim_takes_the_older_batch_first(rows, claim):
    assert capi.load().shrike_expert_reader_claim_slot(_slots(rows), len(rows)) == claim
    assert HL.reader_claim_slot(rows) == claim


@pytest.mark.parametrize("rows,free", [  # publishFindsNoSlotWhileBothAreActive (+BatchDepth.swift:82-100)
    ([(1, 1, 0, 1), (1, 2, 0, 1)], -1), ([(1, 1, 0, 1), (0, 0, 0, 0)], 1), ([(0, 0, 0, 0), (1, 1, 0, 1)], 0)])
def test_publish_finds_the_first_free_slot(rows, free):
    assert capi.load().shrike_expert_reader_free_slot(_slots(rows), len(rows)) == free
    assert HL.reader_free_slot(rows) == free


@pytest.mark.parametrize("before,after", [  # cancellingAPublishedBatchAccountsOnlyItsUnclaimedReads (:146-166)
    ((5, 2, 5, 0), (5, 5, 2, errno.ECANCELED)), ((4, 1, 4, errno.EIO), (4, 4, 1, errno.EIO)), ((3, 3, 1, 0), (3, 3, 1, 0))])
def test_cancel_accounts_only_unclaimed_reads(before, after):
    state = capi.ExpertBatchCancelState(*before)
    capi.load().shrike_expert_reader_cancel_slot(C.byref(state))
    assert (state.count, state.next_index, state.outstanding, state.first_errno) == after
    assert HL.reader_cancel_slot(*before, errno.ECANCELED) == after
