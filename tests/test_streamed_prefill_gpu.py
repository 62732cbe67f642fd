"""A prefill chunk whose experts do not fit the pool: the routed tile loop (scheduler + sequencer) drives
slot-cache plans, reads from a packed layer file and the grouped FFN tile by tile. Every partial row and
the reduced output equal, byte for byte, those of the same chunk with every expert resident."""
import numpy as np
import pytest

from oracle import oracle as O
from shrike_amd import capi, host
from shrike_amd import synth as S
from harness import runners
from tests.helpers import Layer, assert_rel_close
from tests.test_decode_gpu import DeviceLayer
from tests.test_prefill_gpu import token_rows

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("slots,depth,width,lookahead", [(12, 1, 1, 0), (16, 2, 1, 1), (24, 2, 2, 1), (9, 1, 1, 1)])
def test_streamed_chunk_equals_the_resident_chunk(gpu, tmp_path, slots, depth, width, lookahead):
    d, f, ne, k, t = 256, 128, 40, 4, 48
    L = Layer(0x5EED0061, d, f, ne, k, bits=4)
    x = token_rows(L, t, d)

    # the same chunk with all experts resident: one grouping, one grouped FFN
    full = DeviceLayer(gpu, L)
    pf = gpu.Prefill(full.moe)
    hidden = gpu.dev(x)
    idx, w = gpu.empty(4 * t * k), gpu.empty(2 * t * k)
    ws = gpu.empty(pf.router_workspace_bytes(t, ne, d))
    pf.encode_block(full.router_w, None, None, hidden, full.eff_scale, full.expert_scale, full.logit_bias, idx, w, ws, t, ne, d, k, d)
    routes = gpu.GroupedRoutesDevice(t * k, ne)
    pf.group_pairs(idx, w, t, k, ne, routes, residency=full.pool.table)
    want_partials = gpu.empty(2 * t * k * d)
    pf.encode_grouped_expert_gemms(full.pool, full.off, routes, hidden, d, want_partials,
                                   gpu.empty(pf.ffn_workspace_bytes(t, routes.max_row_tiles)), t, k)
    want_h2 = gpu.empty(2 * t * d)
    pf.encode_reduce_token_major(want_partials, w, want_h2, t, k, d)
    gpu.synchronize()
    want_idx = idx.download(np.uint32, t * k)
    used = sorted(set(want_idx.tolist()))
    assert len(used) > slots, "the chunk must need more experts than the pool has cells"

    # the layer file, the reader over it, a pool of `slots` cells and its cache
    S.write_packed_experts(str(tmp_path), [L.blobs], d, f, 4, False)
    layout = host.PackedExpertsLayout.load(str(tmp_path))
    stride = layout.expert_stride
    reader = host.ParallelExpertReader(str(tmp_path / "packed_experts" / layout.layer(0)["file"]), stride, threads=4, batch_depth=2)
    small = DeviceLayer(gpu, L, cells=slots, resident=[])
    small.pool = gpu.ExpertPool(slots, stride, ne)
    small.moe.stream = gpu.Stream()
    cache = host.SlotCache(slots, ne)
    config = host.TileSchedulerConfig(max_pending_depth=depth, tile_experts=8, tiles_per_command_buffer=width,
                                      fetch_lookahead=lookahead)
    layer = runners.StreamedPrefillLayer(small.moe, small.pool, cache, layout.expert_offsets(0, False), reader,
                                     [layout.expert(0, e)["offset"] for e in range(ne)], stride, gpu.PinnedBuffer(4 * stride), t, config)
    assert layer.config.fits_slot_budget(slots)
    router = dict(weights=small.router_w, eff_scale=small.eff_scale, expert_scale=small.expert_scale, bias=small.logit_bias)
    h2 = layer.run(router, hidden, t, d)
    small.moe.stream.synchronize()

    assert np.array_equal(layer.idx.download(np.uint32, t * k), want_idx)
    assert np.array_equal(layer.partials.download(np.uint16, t * k * d), want_partials.download(np.uint16, t * k * d))
    assert np.array_equal(h2.download(np.uint16, t * d), want_h2.download(np.uint16, t * d))

    # and against the oracle, a few pairs
    off = L.oracle_offsets()
    got = layer.partials.download(np.uint16, t * k * d).reshape(t, k, d)
    for tok in (0, t // 2, t - 1):
        xt = np.ascontiguousarray(x[tok * d:(tok + 1) * d])
        for rank in range(k):
            ref = O.prefill_pair_partial(L.blobs[int(want_idx[tok * k + rank])], off, xt, d, f, 4, L.meta)
            assert_rel_close(got[tok, rank], ref, f"token {tok} rank {rank}")

    # the loop did what the sequencer prescribes
    tiles = len(layer.grouped.tiles)
    calls = [c for c, _ in layer.trace]
    assert tiles == -(-len(used) // layer.config.tile_experts) and tiles >= 2
    assert [tl for c, tl in layer.trace if c == "encode"] == list(range(tiles))
    assert [tl for c, tl in layer.trace if c == "begin"] == list(range(tiles))
    assert calls.count("commit") == calls.count("drain") or calls.count("drain") >= calls.count("commit")
    assert "abandonBegun" not in calls
    if lookahead and layer.config.fetch_lookahead:
        first_encode = layer.trace.index(("encode", 0))
        assert ("begin", 1) in layer.trace[:first_encode], "the successor's fetch was not begun before the tile was awaited"
    st = cache.statistics(stride)
    assert st.requested_experts == len(used) and st.misses == len(used) and st.hits == 0
    assert st.loading_slots == 0 and st.resident_slots == min(slots, len(used))
    assert [small.pool.entry(e) for e in range(ne)] == [cache.entry(e) for e in range(ne)]

    # a second chunk over the same tokens: what the last tiles left in the pool is hit, the bytes are the same
    layer.run(router, hidden, t, d)
    small.moe.stream.synchronize()
    assert cache.statistics().hits > 0
    assert np.array_equal(layer.partials.download(np.uint16, t * k * d), want_partials.download(np.uint16, t * k * d))


def test_a_failed_read_ends_the_chunk_and_leaves_no_slot_loading(gpu, tmp_path):
    """A read past the end of the layer file fails one tile's fetch: the sequencer waits out what was begun
    (abandonBegunFetches), the error reaches the caller, and every slot the failed plan had reserved is free."""
    d, f, ne, k, t, slots = 256, 128, 40, 4, 48, 12
    L = Layer(0x5EED0062, d, f, ne, k, bits=4)
    x = token_rows(L, t, d)
    S.write_packed_experts(str(tmp_path), [L.blobs], d, f, 4, False)
    layout = host.PackedExpertsLayout.load(str(tmp_path))
    stride = layout.expert_stride
    reader = host.ParallelExpertReader(str(tmp_path / "packed_experts" / layout.layer(0)["file"]), stride, threads=2)
    small = DeviceLayer(gpu, L, cells=slots, resident=[])
    small.pool = gpu.ExpertPool(slots, stride, ne)
    small.moe.stream = gpu.Stream()
    cache = host.SlotCache(slots, ne)
    offsets = [layout.expert(0, e)["offset"] for e in range(ne)]
    ids, _, _ = O.prefill_router(L.router_dict(), x, t, d, k)
    victim = sorted(set(ids.tolist()))[-1]       # in the chunk's last tile
    offsets[victim] = ne * stride                 # past the end of the file
    layer = runners.StreamedPrefillLayer(small.moe, small.pool, cache, layout.expert_offsets(0, False), reader, offsets, stride,
                                     gpu.PinnedBuffer(4 * stride), t, host.TileSchedulerConfig(2, 8, 1, 1))
    router = dict(weights=small.router_w, eff_scale=small.eff_scale, expert_scale=small.expert_scale, bias=small.logit_bias)
    with pytest.raises(capi.ShrikeError, match="expert read failed"):
        layer.run(router, gpu.dev(x), t, d)
    small.moe.stream.synchronize()
    calls = [c for c, _ in layer.trace]
    assert calls[-1] == "abandonBegun" and calls.count("encode") >= 1
    st = cache.statistics(stride)
    assert st.loading_slots == 0
    assert victim not in cache.resident_experts()
