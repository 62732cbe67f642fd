"""The operators under HIP graph capture: a captured sequence replayed several times, with eager work and
synchronisations of the program's own between the replays and other inputs for every replay, gives on every replay the
bytes the same calls give eagerly. (The benchmark's figures come from such graphs.)"""
import ctypes as C

import numpy as np
import pytest

from shrike_amd import capi
from shrike_amd import synth as S
from tests.helpers import Layer
from tests.test_decode_gpu import DeviceLayer

pytestmark = pytest.mark.gpu


def capture(gpu, stream, body):
    capi.check(capi.load().shrike_hip_graph_begin_capture(stream.handle), "graph_begin_capture")
    body()
    graph = capi.load().shrike_hip_graph_end_capture(stream.handle)
    assert graph, capi.last_error()
    return graph


def outputs(dl, d, k, f):
    return (dl.y.download(np.uint16, d), dl.hidden.download(np.uint16, d), dl.out_idx.download(np.uint32, k),
            dl.out_w.download(np.uint16, k), dl.acts.download(np.uint16, k * f))


@pytest.mark.parametrize("entry", ["layer", "noalloc", "norm"])
def test_decode_layer_replays_equal_eager_calls(gpu, entry):
    d, f, ne, k = 2048, 512, 64, 8
    L = Layer(0x5EED0C01, d, f, ne, k, shared_f=512)
    dl = DeviceLayer(gpu, L)
    stream = gpu.Stream()
    dl.moe.stream = stream
    args = dl.layer_args()
    delta = weight = None
    if entry == "norm":  # the residual add + RMS norm in the layer's first launch: x is written by the call
        delta = gpu.dev(S.f32_to_f16_bits(L.tree.key("delta").normal(d, std=0.05)))
        weight = gpu.dev(S.f32_to_bf16_bits(L.tree.key("norm.w").uniform(0.5, 1.5, d)))
        args.norm_delta, args.norm_weight, args.norm_eps = delta.ptr, weight.ptr, 1e-6

    def call():
        if entry == "noalloc":
            capi.check(capi.load().shrike_hip_moe_decode_layer_noalloc(C.byref(dl.moe.desc), stream.handle, C.byref(args)),
                       "shrike_hip_moe_decode_layer_noalloc")
        else:
            dl.moe.encode_decode_layer(args)

    graph = capture(gpu, stream, call)
    other = gpu.empty(1 << 16)
    try:
        for replay in range(5):
            x = S.f32_to_f16_bits(L.tree.key(f"replay.x.{replay}").normal(d, std=1.0))
            hidden = S.f32_to_f16_bits(L.tree.key(f"replay.hidden.{replay}").normal(d, std=1.0))
            # eagerly first
            dl.x.upload(x)
            dl.hidden.upload(hidden)
            call()
            stream.synchronize()
            want = outputs(dl, d, k, f)
            # unrelated eager work, then the replay over the same inputs
            other.fill(replay)
            dl.x.upload(x)
            dl.hidden.upload(hidden)
            for b in (dl.y, dl.out_idx, dl.out_w, dl.acts):
                b.fill(0x5A)
            capi.check(capi.load().shrike_hip_graph_launch(graph, stream.handle), "graph_launch")
            stream.synchronize()
            got = outputs(dl, d, k, f)
            for name, a, b in zip(("y", "hidden", "indices", "weights", "acts"), got, want):
                assert np.array_equal(a, b), f"replay {replay}: {name} differs from the eager call"
    finally:
        capi.check(capi.load().shrike_hip_graph_destroy(graph), "graph_destroy")


def test_prefill_chunk_replays_equal_eager_calls(gpu):
    d, f, ne, k, t = 512, 256, 32, 4, 96
    L = Layer(0x5EED0C02, d, f, ne, k)
    dl = DeviceLayer(gpu, L)
    stream = gpu.Stream()
    dl.moe.stream = stream
    pf = gpu.Prefill(dl.moe)
    hidden = gpu.empty(2 * t * d)
    idx, w, ws = gpu.empty(4 * t * k), gpu.empty(2 * t * k), gpu.empty(pf.router_workspace_bytes(t, ne, d))
    routes = gpu.GroupedRoutesDevice(t * k, ne)
    partials, h2 = gpu.empty(2 * t * k * d), gpu.empty(2 * t * d)
    work = gpu.empty(pf.ffn_workspace_bytes(t, routes.max_row_tiles))

    def chunk():
        pf.encode_block(dl.router_w, dl.router_s, dl.router_b, hidden, dl.eff_scale, dl.expert_scale, dl.logit_bias, idx, w, ws,
                        t, ne, d, k, d)
        pf.group_pairs(idx, w, t, k, ne, routes, residency=dl.pool.table)
        pf.encode_grouped_expert_gemms(dl.pool, dl.off, routes, hidden, d, partials, work, t, k)
        pf.encode_reduce_token_major(partials, w, h2, t, k, d)

    graph = capture(gpu, stream, chunk)
    try:
        for replay in range(4):
            rows = S.f32_to_f16_bits(L.tree.key(f"replay.rows.{replay}").normal(t * d, std=1.0))
            hidden.upload(rows)
            chunk()
            stream.synchronize()
            want = (idx.download(np.uint32, t * k), h2.download(np.uint16, t * d))
            hidden.upload(rows)
            for b in (idx, h2, partials):
                b.fill(0x5A)
            capi.check(capi.load().shrike_hip_graph_launch(graph, stream.handle), "graph_launch")
            stream.synchronize()
            assert np.array_equal(idx.download(np.uint32, t * k), want[0]), f"replay {replay}: routes"
            assert np.array_equal(h2.download(np.uint16, t * d), want[1]), f"replay {replay}: reduced rows"
    finally:
        capi.check(capi.load().shrike_hip_graph_destroy(graph), "graph_destroy")
