"""The allocation-free decode-layer entry point against the entry point it is a variant of: same routes, same
bytes out, on calls in a row that share the library's static scratch (the second smaller than the first, the
third with experts missing from the pool so that stale activations of earlier calls sit where nothing may read)."""
import ctypes as C

import numpy as np
import pytest

from shrike_amd import capi
from tests.helpers import Layer
from tests.test_decode_gpu import DeviceLayer

pytestmark = pytest.mark.gpu

SCRATCH_FIELDS = ("resolved_slots", "hit_count", "hit_positions", "miss_count", "miss_positions", "miss_experts",
                  "acts", "shared_scratch", "h1")


def run_both(gpu, L, resident=None, bind_lists=False, stream=None):
    d, k = L.d, L.k
    dl = DeviceLayer(gpu, L, resident=resident)
    dl.moe.encode_decode_layer(dl.layer_args())
    gpu.synchronize()
    want = dict(y=dl.y.download(np.uint16, d), hidden=dl.hidden.download(np.uint16, d),
                idx=dl.out_idx.download(np.uint32, k), w=dl.out_w.download(np.uint16, k),
                resolved=dl.resolved.download(np.uint32, k), misses=int(dl.miss_count.download(np.uint32, 1)[0]))
    # the variant: fresh residual stream, outputs pre-filled with a pattern, no scratch from the caller
    dl.hidden.upload(L.hidden)
    for b in (dl.y, dl.out_idx, dl.out_w, dl.resolved, dl.miss_count):
        b.fill(0xA5)
    args = dl.layer_args()
    for name in SCRATCH_FIELDS:
        if not (bind_lists and name in ("resolved_slots", "miss_count")):
            setattr(args, name, None)
    # what the entry point exists for: device memory is not allocated (or freed) by the call. The first call of the
    # process has looked the scratch's address up already (shrike_hip_init does), so every call is held to it.
    lib = capi.load()
    free_before, free_after = C.c_uint64(0), C.c_uint64(0)
    gpu.synchronize()
    capi.check(lib.shrike_hip_mem_info(C.byref(free_before), None), "shrike_hip_mem_info")
    capi.check(lib.shrike_hip_moe_decode_layer_noalloc(C.byref(dl.moe.desc), stream.handle if stream else None, C.byref(args)),
               "shrike_hip_moe_decode_layer_noalloc")
    capi.check(lib.shrike_hip_mem_info(C.byref(free_after), None), "shrike_hip_mem_info")
    assert free_after.value == free_before.value, "the allocation-free entry point changed the device's free memory"
    gpu.synchronize()
    assert np.array_equal(dl.out_idx.download(np.uint32, k), want["idx"])
    assert np.array_equal(dl.out_w.download(np.uint16, k), want["w"])
    assert np.array_equal(dl.y.download(np.uint16, d), want["y"])
    assert np.array_equal(dl.hidden.download(np.uint16, d), want["hidden"])
    if bind_lists:
        assert np.array_equal(dl.resolved.download(np.uint32, k), want["resolved"])
        assert int(dl.miss_count.download(np.uint32, 1)[0]) == want["misses"]
    return want


def test_the_allocation_free_layer_equals_the_layer_entry_point(gpu):
    big = Layer(0x5EED0701, 2048, 512, 64, 8, shared_f=512)
    small = Layer(0x5EED0702, 512, 256, 32, 4, bits=8, shared_f=256, shared_bits=8)
    run_both(gpu, big)
    run_both(gpu, small)  # a smaller call right behind a larger one, in the same scratch
    # experts missing from the pool: their positions are skipped, whatever earlier calls left in the scratch
    want = run_both(gpu, big, resident=[e for e in range(64) if e % 3], bind_lists=True)
    assert 0 < want["misses"] < 8
    no_shared = Layer(0x5EED0703, 2880, 192, 32, 4, router_bits=8)
    run_both(gpu, no_shared)
    run_both(gpu, small, stream=gpu.Stream())  # on a stream of the caller's: the scratch is the stream's device's


def test_the_allocation_free_layer_rejects_what_its_scratch_cannot_hold(gpu):
    L = Layer(0x5EED0704, 128, 64, 16, 4)
    dl = DeviceLayer(gpu, L)
    args = dl.layer_args()
    lib = capi.load()
    desc = capi.MoEDesc(128, 4096 + 64, 16, 4, 4, 0, capi.META_BF16, capi.ACT_SILU, 0, 0, 1.0, 0)
    assert lib.shrike_hip_moe_decode_layer_noalloc(C.byref(desc), None, C.byref(args)) != 0
    assert "static scratch" in capi.last_error()
    desc = capi.MoEDesc(128, 64, 16, 9, 4, 0, capi.META_BF16, capi.ACT_SILU, 0, 0, 1.0, 0)
    assert lib.shrike_hip_moe_decode_layer_noalloc(C.byref(desc), None, C.byref(args)) != 0
    assert "topK" in capi.last_error()
    assert lib.shrike_hip_moe_decode_layer_noalloc(None, None, C.byref(args)) != 0
