"""The host-only exports that have no device side: the CPU expert kernel (shrike_int4_affine_gemv,
CPUExpertFFN.accumulate) against the reference's own committed vectors and the oracle, the host's half of
the tagged router readback on the vectors of RouterHostReadbackTests.swift, and the completion timeline on
the cases of ExpertLoadOperationTests.swift."""
import ctypes as C
import json
import os
import zlib

import numpy as np
import pytest

from oracle import oracle as O
from shrike_amd import capi
from shrike_amd import host as HL
from shrike_amd import synth as S

HERE = os.path.dirname(os.path.abspath(__file__))


def test_int4_gemv_export_gives_the_reference_c_bits():
    """tests/golden/ref_int4_gemv.json holds what the reference's C kernel returned for these seeded inputs."""
    from tests.golden.make_ref_gemv_vectors import inputs
    cases = json.load(open(os.path.join(HERE, "golden", "ref_int4_gemv.json")))["cases"]
    assert len(cases) >= 3
    for case in cases:
        rows, n = case["rows"], case["n"]
        w, s, b, x = inputs(rows, n)
        y = HL.int4_affine_gemv(w, s, b, x, rows, n).view(np.uint32)
        assert [int(v) for v in y[:16]] == case["head"], (rows, n)
        assert zlib.crc32(y.tobytes()) == case["crc32"], (rows, n)


@pytest.mark.parametrize("rows,n", [(1, 64), (3, 128), (7, 8192), (33, 2880)])  # 8192: more groups than the stack buffer holds
def test_int4_gemv_export_equals_the_oracle_and_the_definition(rows, n):
    tree = S.SeedTree(0xA11 + rows + n)
    w, s, b = S.affine_matrix(tree.key("w"), rows, n, 4, S.META_BF16)
    x = tree.key("x").normal(n).astype(np.float32)
    y = HL.int4_affine_gemv(w, s, b, x, rows, n)
    assert np.array_equal(y.view(np.uint32), O.int4_affine_gemv(w, s, b, x, rows, n, S.META_BF16).view(np.uint32))
    # the format's definition in fp64: w = q * s + b, low nibble = even element
    q = np.stack([w.reshape(rows, n // 2) & 0x0F, w.reshape(rows, n // 2) >> 4], axis=-1).reshape(rows, n).astype(np.float64)
    sf = np.repeat(S.bf16_bits_to_f32(s).reshape(rows, n // 64).astype(np.float64), 64, axis=1)
    bf = np.repeat(S.bf16_bits_to_f32(b).reshape(rows, n // 64).astype(np.float64), 64, axis=1)
    want = ((q * sf + bf) * x.astype(np.float64)).sum(axis=1)
    assert np.max(np.abs(y - want)) <= 1e-5 * max(1.0, np.max(np.abs(want))) + 1e-4


def test_cpu_expert_ffn_accumulate_equals_the_oracle_bit_for_bit_and_accumulates():
    d, f = 2048, 512
    tree = S.SeedTree(0xA11F)
    blob = S.expert_blob(tree, "expert", d, f, 4, S.META_BF16)
    off = capi.ExpertOffsets()
    assert capi.load().shrike_expert_offsets_make(d, f, 4, 0, off) == blob.nbytes == 1_769_472
    o_off, _ = O.expert_offsets(d, f, 4)
    x = tree.key("x").normal(d).astype(np.float32)
    out = np.zeros(d, np.float32)
    HL.cpu_expert_ffn_accumulate(blob, off, x, d, f, 0.25, out)
    want = np.zeros(d, np.float32)
    O.cpu_expert_ffn_accumulate(blob, o_off, x, d, f, 0.25, want, bits=4, meta=S.META_BF16)
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    assert np.any(out != 0)
    # a second call accumulates (CPUExpertFFNTests: accumulate twice = twice the single result for weight w)
    once = out.copy()
    HL.cpu_expert_ffn_accumulate(blob, off, x, d, f, 0.25, out)
    assert np.array_equal(out, once + once)
    # scratch sized by the library; a NULL or a ragged shape is EINVAL, not a crash
    assert capi.load().shrike_cpu_expert_ffn_scratch_floats(d, f) == 2 * f + d
    with pytest.raises(capi.ShrikeError):
        HL.cpu_expert_ffn_accumulate(blob, off, x, d, 100, 0.25, out)


# ---------------------------------------------------------------- RouterHostReadbackTests.swift:18-91

TOP_K = 4


def readback_words(tag, hit_count=3, miss_count=1, ids=(5, 9, 200, 3), weight_bits=(0x3c00, 0x3800, 0x3400, 0x3000),
                   hit_positions=(0, 2, 3, 0), miss_positions=(1, 0, 0, 0), predicted=(1, 2, 3, 4)):
    values = [hit_count, miss_count, *ids, *weight_bits, *hit_positions, *miss_positions, *predicted]
    return np.array([HL.RouterHostReadback.word(tag, v) for v in values], np.uint32)


def test_readback_word_count_covers_the_counts_and_five_top_k_runs():
    assert HL.RouterHostReadback.word_count(4) == 22 and HL.RouterHostReadback.word_count(8) == 42


def test_readback_decode_reads_counts_ids_weights_and_positions():
    words = readback_words(7)
    got = HL.RouterHostReadback.decode(words.ctypes.data, TOP_K, 7)
    assert got == dict(hit_count=3, miss_count=1, expert_ids=[5, 9, 200, 3], weight_bits=[0x3c00, 0x3800, 0x3400, 0x3000],
                       hit_positions=[0, 2, 3], miss_positions=[1], predicted_ids=[1, 2, 3, 4])
    assert HL.RouterHostReadback.is_complete(words.ctypes.data, TOP_K, 7)


def test_readback_decode_returns_none_until_every_word_carries_the_tag():
    words = readback_words(7)
    words[HL.RouterHostReadback.word_count(TOP_K) - 1] = HL.RouterHostReadback.word(6, 4)
    assert not HL.RouterHostReadback.is_complete(words.ctypes.data, TOP_K, 7)
    assert HL.RouterHostReadback.decode(words.ctypes.data, TOP_K, 7) is None
    zeroed = np.zeros(HL.RouterHostReadback.word_count(TOP_K), np.uint32)
    assert not HL.RouterHostReadback.is_complete(zeroed.ctypes.data, TOP_K, 1)
    # a middle word stale
    words = readback_words(7)
    words[2 + TOP_K + 1] = HL.RouterHostReadback.word(6, 0x3800)
    assert HL.RouterHostReadback.decode(words.ctypes.data, TOP_K, 7) is None
    # only the counts tagged
    words = np.zeros(HL.RouterHostReadback.word_count(TOP_K), np.uint32)
    words[0], words[1] = HL.RouterHostReadback.word(7, 3), HL.RouterHostReadback.word(7, 1)
    assert not HL.RouterHostReadback.is_complete(words.ctypes.data, TOP_K, 7)
    assert HL.RouterHostReadback.decode(words.ctypes.data, TOP_K, 7) is None


def test_readback_decode_clamps_counts_to_top_k_and_tags_skip_zero():
    got = HL.RouterHostReadback.decode(readback_words(3, hit_count=9, miss_count=9).ctypes.data, TOP_K, 3)
    assert got["hit_count"] == 4 and got["miss_count"] == 4 and len(got["hit_positions"]) == 4
    assert [HL.RouterHostReadback.next_tag(t) for t in (0, 5, 0xffff)] == [1, 6, 1]


def test_readback_poll_sees_words_another_thread_writes_and_gives_up_at_the_deadline():
    import threading
    import time
    count = HL.RouterHostReadback.word_count(TOP_K)
    words = np.zeros(count, np.uint32)
    assert HL.RouterHostReadback.poll(words.ctypes.data, TOP_K, 9, 2_000_000) is None  # 2 ms: nothing arrives
    fresh = readback_words(9)

    def writer():
        for i in reversed(range(count)):  # payload first, counts last, a word at a time
            time.sleep(0.0005)
            words[i] = fresh[i]
    t = threading.Thread(target=writer)
    t.start()
    got = HL.RouterHostReadback.poll(words.ctypes.data, TOP_K, 9, 2_000_000_000)
    t.join()
    assert got is not None and got["expert_ids"] == [5, 9, 200, 3] and got["miss_positions"] == [1]


# ---------------------------------------------------------------- ExpertLoadOperationTests.swift:95-150

def test_timeline_does_not_advance_past_an_out_of_order_batch():
    timeline = HL.ExpertIOTimeline()
    first, second = timeline.reserve(), timeline.reserve()
    assert (first.value, second.value) == (1, 2) and first.status[0] == 0 and second.status[0] == 0
    assert timeline.publish(second, True) == 0
    assert second.status[0] == 1 and timeline.published == 0
    assert timeline.publish(first, True) == second.value == timeline.published


def test_timeline_failed_batch_is_terminal():
    timeline = HL.ExpertIOTimeline()
    token = timeline.reserve()
    assert timeline.publish(token, False) == token.value
    assert token.status[0] == 2


def test_timeline_status_words_recycle_after_one_ring_of_values():
    ring = np.full(4096, 0xFFFFFFFF, np.uint32)  # caller-owned words, as pinned memory would be
    timeline = HL.ExpertIOTimeline(ring.ctypes.data)
    first = timeline.reserve()
    assert ring[0] == 0
    for _ in range(1, 4096):
        timeline.publish(timeline.reserve(), True)
    assert timeline.published == 0  # everything is held behind the first value
    timeline.publish(first, False)
    assert timeline.published == 4096 and ring[0] == 2 and np.all(ring[1:] == 1)
    recycled = timeline.reserve()
    assert recycled.value == first.value + 4096 and recycled.status_index == first.status_index == 0
    assert ring[0] == 0
    assert timeline.publish(recycled, True) == recycled.value


def test_timeline_under_concurrent_publishers_ends_at_the_last_value():
    import threading
    timeline = HL.ExpertIOTimeline(word_count=64)
    tokens = [timeline.reserve() for _ in range(400)]
    assert [t.value for t in tokens] == list(range(1, 401))

    def publish(part):
        for token in part:
            timeline.publish(token, True)
    threads = [threading.Thread(target=publish, args=(tokens[i::4][::-1],)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert timeline.published == 400
