#!/usr/bin/env python3
"""Benchmark of the routed-expert decode layer on one MI355X.

A step is one MoE-layer decode for one token at the 35B-A3B int4 shape (hidden 2048,
256 routed experts of intermediate 512, top-8, one shared expert of intermediate 512,
fp16 router, group-64 affine int4 with 16-bit scale/bias): router -> top-k -> slot
resolve -> shared expert -> gate/up matvec + SiLU-multiply -> down matvec + weighted
combine. Consecutive steps walk a stack of 40 layers whose expert pools sit at distinct
addresses (18 GB, far past the 256 MB Infinity Cache), and the activation vector rotates
over four variants so that a layer picks other experts from one pass to the next: every
step streams its experts from HBM. Runs of layers are captured in HIP graphs.

Timing: W warm-up steps, then REGIONS regions of exactly K steps each in one captured
graph, the device clock stored by a one-thread kernel between regions (HIP events on the
launch stream bracket the whole graph as the cross-check, and bracket every region where
the clock is not to be had); `ms_per_step` is the median region / K (minimum and maximum
are reported beside it, and what two stamps with nothing between them measure).

Prints ONE JSON line. `value` is expert bytes read per second (8 routed + 1 shared
expert = 15,925,248 B per step) with all inputs resident in HBM. `roofline` prices the
dominant kernel of the timed layer (its second launch) against 8 TB/s; `cpu_baseline`
times the CPU oracle's fp32 port on this host (the layer on several cores, and one
expert on one core); `secondary` carries the other workloads of the benchmark
definition (ragged prefill chunk, gpt-oss-shape batch, Kimi-shape batch through a
64-of-256 pool), each measured by the same run.
"""
from __future__ import annotations

import argparse
import ctypes as C
import gc
import json
import os
import re
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

D, F, NE, K, FS, BITS = 2048, 512, 256, 8, 512, 4
HBM_PEAK_GBPS = 8000.0
REGIONS = 15          # timed regions; the median is reported
CHASE_HOPS = 64       # dependent loads in the round-trip probe
X_VARIANTS = 4        # activation vectors in rotation
PROFILES = os.path.join(ROOT, "profiles")


# Under rocprofv3 a run of --steps 2000 once ended in an abort inside hipGraphLaunch (an earlier form of this file: one
# executable graph of 120 kernel nodes launched fifty times back to back). Its cause was never shown, so a profiled run
# is held to what has run clean under the profiler: at most this many steps a region.
PROFILED_MAX_STEPS = 400


def profiler_attached() -> bool:
    env = os.environ
    named = " ".join(env.get(k, "") for k in ("LD_PRELOAD", "ROCP_TOOL_LIBRARIES", "HSA_TOOLS_LIB", "ROCPROFILER_LIBRARY_PATH"))
    return "rocprof" in named.lower() or any(k.startswith(("ROCPROF_", "ROCPROFILER_")) for k in env)


def profile_figure(filename: str, key: str):
    """A figure from a tracked rocprofv3 summary: the first line `key: <number>`; None when absent."""
    try:
        with open(os.path.join(PROFILES, filename)) as fh:
            for line in fh:
                m = re.match(r"\s*" + re.escape(key) + r"\s*:\s*([0-9][0-9_,.]*)", line)
                if m:
                    return int(float(m.group(1).replace(",", "").replace("_", "")))
    except OSError:
        pass
    return None


def build_layers(rt, capi, S, n_layers, meta, shared=True):
    """Layer 0's pool comes from the seeded generator; the other layers hold byte copies of it at
    their own addresses (cache behaviour follows addresses, not values). Routers, shared experts
    and activations are distinct per layer."""
    tree = S.SeedTree(0x5EED0002)
    off, stride = rt.expert_offsets(D, F, BITS)
    t0 = time.time()
    blobs = [S.expert_blob(tree, f"layer.0.expert.{e}", D, F, BITS, meta) for e in range(NE)]
    layers = []
    ones_d = rt.dev(S.f32_to_bf16_bits(np.ones(D, np.float32)))
    ones_e = rt.dev(S.f32_to_bf16_bits(np.ones(NE, np.float32)))
    zeros_e = rt.dev(np.zeros(NE, np.uint16))
    hidden = rt.dev(S.activations_f16(tree, "hidden", D))
    first_pool = None
    # the decode scratch is one set of buffers for all layers, as in the reference's runner
    # (sources/Shrike/Runtime/Inference/RealForwardRunner.swift:754-825)
    scratch = {name: rt.empty(size) for name, size in dict(idx=32, w=16, res=32, hc=4, hp=32, mc=4, mp=32, me=32,
                                                           acts=2 * K * F, ss=4 * FS, h1=2 * D, y=2 * D).items()}
    xs = [rt.dev(S.activations_f16(tree, "layer.x" if v == 0 else f"layer.x.{v}", D)) for v in range(X_VARIANTS)]
    for l in range(n_layers):
        pool = rt.ExpertPool(NE, stride, NE)
        if l == 0:
            for e in range(NE):
                capi.check(capi.load().shrike_hip_memcpy_h2d(pool.cell_ptr(e), blobs[e].ctypes.data, blobs[e].nbytes), "h2d")
            first_pool = pool
        else:
            capi.check(capi.load().shrike_hip_memcpy_d2d(pool.cell_ptr(0), first_pool.cell_ptr(0), NE * pool.stride), "d2d")
        for e in range(NE):
            pool.publish(e, e, capi.RESIDENT)
        lay = dict(pool=pool, x=xs[0], xs=xs, **scratch)
        lay["router"] = rt.dev(S.router_f16(tree, f"layer.{l}.router.w", NE, D))
        lay["shared"] = {n: tuple(rt.dev(t) for t in S.affine_matrix(tree.key(f"layer.{l}.shared.{n}"), r, c, BITS, meta))
                         for n, r, c in (("gate", FS, D), ("up", FS, D), ("down", D, FS))}
        a = capi.DecodeLayerArgs()
        a.router_weights, a.effective_scale, a.per_expert_scale, a.logit_bias = lay["router"].ptr, ones_d.ptr, ones_e.ptr, zeros_e.ptr
        a.pool, a.pool_slot_stride, a.residency, a.offsets = pool.bases, pool.stride, pool.table, off
        for n in ("gate", "up", "down"):
            if shared:
                setattr(a, f"shared_{n}", capi.Projection(*(t.ptr for t in lay["shared"][n])))
        a.shared_bits, a.shared_f = BITS, FS
        a.x, a.hidden, a.y = lay["x"].ptr, hidden.ptr, lay["y"].ptr
        a.out_indices, a.out_weights, a.resolved_slots = lay["idx"].ptr, lay["w"].ptr, lay["res"].ptr
        a.hit_count, a.hit_positions, a.miss_count = lay["hc"].ptr, lay["hp"].ptr, lay["mc"].ptr
        a.miss_positions, a.miss_experts = lay["mp"].ptr, lay["me"].ptr
        a.acts, a.shared_scratch, a.h1 = lay["acts"].ptr, lay["ss"].ptr, lay["h1"].ptr
        lay["args"] = a
        lay["args_x"] = [a]
        for v in range(1, X_VARIANTS):  # the same layer over another activation vector
            b = capi.DecodeLayerArgs()
            C.memmove(C.byref(b), C.byref(a), C.sizeof(b))
            b.x = xs[v].ptr
            lay["args_x"].append(b)
        layers.append(lay)
    rt.synchronize()
    keep = (ones_d, ones_e, zeros_e, hidden, blobs)
    return layers, off, stride, keep, time.time() - t0


def capture(rt, capi, stream, body):
    capi.check(capi.load().shrike_hip_graph_begin_capture(stream.handle), "graph_begin_capture")
    try:
        body()
    except Exception:
        broken = capi.load().shrike_hip_graph_end_capture(stream.handle)  # the stream must leave capture mode
        if broken:
            capi.load().shrike_hip_graph_destroy(broken)
        raise
    g = capi.load().shrike_hip_graph_end_capture(stream.handle)
    if not g:
        raise capi.ShrikeError(capi.last_error())
    return g


def time_graph(rt, capi, stream, graph, launches):
    start, stop = rt.Event(), rt.Event()
    stream.synchronize()
    rt.synchronize()
    start.record(stream)
    for _ in range(launches):
        capi.check(capi.load().shrike_hip_graph_launch(graph, stream.handle), "graph_launch")
    stop.record(stream)
    stop.synchronize()
    rt.synchronize()
    return start.elapsed_ms(stop)


def median_of_regions(rt, capi, stream, graph, launches, regions=REGIONS):
    """ms per launch of `graph`: the median over `regions` event-bracketed regions of `launches` launches each."""
    events = [rt.Event() for _ in range(regions + 1)]
    stream.synchronize()
    events[0].record(stream)
    for r in range(regions):
        for _ in range(launches):
            capi.check(capi.load().shrike_hip_graph_launch(graph, stream.handle), "graph_launch")
        events[r + 1].record(stream)
    events[-1].synchronize()
    return statistics.median(events[r].elapsed_ms(events[r + 1]) for r in range(regions)) / launches


class LayerWalk:
    """Exactly-K-step regions over the layer stack: a region is a run of graph launches that covers K consecutive
    layers (wrapping round the stack), each launch over the next activation variant. Graphs are captured once per
    (variant, first layer, layer count)."""

    def __init__(self, rt, capi, moe, stream, layers):
        self.rt, self.capi, self.moe, self.stream, self.layers = rt, capi, moe, stream, layers
        self.graphs = {}
        self.at, self.variant = 0, 0

    def graph(self, variant, first, count):
        key = (variant, first, count)
        if key not in self.graphs:
            def body():
                for lay in self.layers[first:first + count]:
                    self.moe.encode_decode_layer(lay["args_x"][variant])
            self.graphs[key] = capture(self.rt, self.capi, self.stream, body)
        return self.graphs[key]

    def enqueue(self, steps):
        """Enqueues exactly `steps` layers, continuing where the last call stopped."""
        n = len(self.layers)
        while steps > 0:
            count = min(steps, n - self.at)
            g = self.graph(self.variant, self.at, count)
            self.capi.check(self.capi.load().shrike_hip_graph_launch(g, self.stream.handle), "graph_launch")
            self.at = (self.at + count) % n
            self.variant = (self.variant + 1) % X_VARIANTS
            steps -= count

    def encode(self, steps):
        """Encodes exactly `steps` layers on the stream (for a capture that holds several regions), continuing where
        the last call stopped, the activation variant moving on at every wrap of the stack as in enqueue."""
        n = len(self.layers)
        while steps > 0:
            count = min(steps, n - self.at)
            for lay in self.layers[self.at:self.at + count]:
                self.moe.encode_decode_layer(lay["args_x"][self.variant])
            self.at = (self.at + count) % n
            self.variant = (self.variant + 1) % X_VARIANTS
            steps -= count

    def plan(self, steps, regions):
        """Captures what `regions` regions of `steps` steps will launch, so that no capture falls into a timed region."""
        at, variant = self.at, self.variant
        n = len(self.layers)
        for _ in range(regions):
            left = steps
            while left > 0:
                count = min(left, n - at)
                self.graph(variant, at, count)
                at, variant, left = (at + count) % n, (variant + 1) % X_VARIANTS, left - count


def cpu_baseline(S, blobs, sample_layers, meta):
    """The oracle's fp32 port of the layer (one task per expert, as
    sources/Shrike/Kernels/CPU/CPUExpertFFN.swift:10-14 describes) on this host's cores, and config 1 of the
    benchmark definition: one routed expert for one token on one core."""
    from oracle import oracle as O
    off, _ = O.expert_offsets(D, F, BITS)
    cores = min(K + 1, len(os.sched_getaffinity(0)))
    tree = S.SeedTree(0xC0FFEE)
    x = tree.key("x").normal(D)
    rng = np.random.default_rng(0)
    weights = np.full(K + 1, 1.0 / K, np.float32)
    t0 = time.perf_counter()
    for i in range(sample_layers):
        picks = rng.choice(NE, K + 1, replace=False)
        O.cpu_layer_fp32([blobs[int(e)] for e in picks], weights, off, x, D, F, cores, bits=BITS, meta=meta)
    per_layer = (time.perf_counter() - t0) / sample_layers
    expert_bytes = (K + 1) * 1_769_472
    # config 1: one expert, one token, one core (sources/Shrike/Kernels/CPU/CPUExpertFFN.swift:102-140)
    singles = max(8, sample_layers // 2)
    out = np.zeros(D, np.float32)
    picks = rng.choice(NE, singles, replace=True)
    t0 = time.perf_counter()
    for e in picks:
        O.cpu_expert_ffn_accumulate(blobs[int(e)], off, x, D, F, 0.125, out, bits=BITS, meta=meta)
    per_expert = (time.perf_counter() - t0) / singles
    # the library's own host export of the same kernel (shrike_cpu_expert_ffn_accumulate: what a host that keeps experts
    # in CPU memory would call), over blobs with the bf16 metadata the reference's CPU kernel takes
    from shrike_amd import host as HL
    from shrike_amd import capi as _capi
    tree_p = S.SeedTree(0x5EED0001)
    blobs_p = [S.expert_blob(tree_p, f"expert.{e}", D, F, BITS, S.META_BF16) for e in range(8)]
    p_off = _capi.ExpertOffsets()
    _capi.load().shrike_expert_offsets_make(D, F, BITS, 0, p_off)
    p_scratch = np.empty(2 * F + D, np.float32)
    p_out = np.zeros(D, np.float32)
    xp = np.ascontiguousarray(x, np.float32)
    t0 = time.perf_counter()
    for i in range(singles):
        HL.cpu_expert_ffn_accumulate(blobs_p[i % len(blobs_p)], p_off, xp, D, F, 0.125, p_out, p_scratch)
    per_product = (time.perf_counter() - t0) / singles
    # the same with the reference's own shrike_int4_affine_gemv, compiled from its source by oracle/Makefile where the
    # reference checkout was present at build time (three calls and the fp32 SiLU-multiply between them, as
    # CPUExpertFFN.accumulate composes them); its metadata is bf16, so it runs over blobs generated with bf16 metadata
    reference = None
    if O.ref_lib_path() is not None:
        tree_r = S.SeedTree(0x5EED0001)
        blobs_r = [S.expert_blob(tree_r, f"expert.{e}", D, F, BITS, S.META_BF16) for e in range(8)]
        codes, metas = F * D // 2, F * (D // 64) * 2
        down_codes, down_metas = D * F // 2, D * (F // 64) * 2

        def parts(blob):
            at, out = 0, []
            for c, m in ((codes, metas), (codes, metas), (down_codes, down_metas)):
                out.append((blob[at:at + c], blob[at + c:at + c + m].view(np.uint16), blob[at + c + m:at + c + 2 * m].view(np.uint16)))
                at += c + 2 * m
            return out
        split = [parts(b) for b in blobs_r]
        xr = np.ascontiguousarray(x, np.float32)
        acc = np.zeros(D, np.float32)
        t0 = time.perf_counter()
        for i in range(singles):
            (gw, gs, gb), (uw, us, ub), (dw, ds, db) = split[i % len(split)]
            g = O.ref_int4_affine_gemv(gw, gs, gb, xr, F, D)
            u = O.ref_int4_affine_gemv(uw, us, ub, xr, F, D)
            act = (g / (1.0 + np.exp(-g)) * u).astype(np.float32)
            acc += 0.125 * O.ref_int4_affine_gemv(dw, ds, db, act, D, F)
        per_ref = (time.perf_counter() - t0) / singles
        reference = {"kind": "reference", "cores": 1, "us_per_expert": round(per_ref * 1e6, 1),
                     "value": round(1_769_472 / per_ref / 1e9, 3), "unit": "GB/s",
                     "sample": f"{singles} experts, the reference's int4_affine_gemv.c (gcc -std=c99 -O2, portable branch), one thread"}
    return {"value": round(expert_bytes / per_layer / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
            "us_per_layer": round(per_layer * 1e6, 1),
            "sample": f"{sample_layers} layer evaluations of 9 experts (8 routed + 1 shared-sized) drawn from the "
                      f"256-expert pool, fp32 scalar C port of shrike_int4_affine_gemv + CPUExpertFFN.accumulate, "
                      f"{cores} threads, gcc -O2",
            "config1": {"workload": "config 1: one routed expert SwiGLU FFN for one token (hidden 2048, intermediate 512, int4)",
                        "cores": 1, "kind": "port", "us_per_expert": round(per_product * 1e6, 1),
                        "value": round(1_769_472 / per_product / 1e9, 3), "unit": "GB/s", "bytes_per_expert": 1_769_472,
                        "sample": f"{singles} calls of the library's host export shrike_cpu_expert_ffn_accumulate over 8 seeded experts, one thread",
                        "oracle_port": {"us_per_expert": round(per_expert * 1e6, 1), "value": round(1_769_472 / per_expert / 1e9, 3),
                                        "unit": "GB/s", "sample": f"{singles} experts drawn from the pool through the oracle's scalar C, one thread"},
                        **({"reference_c": reference} if reference else {})}}


def cpu_pairs(S, blobs, d, f, bits, meta, pairs, evaluations, label):
    """The oracle's fp32 port of one step's expert FFNs on this host's cores: `pairs` (token, expert) FFN evaluations,
    one task each (sources/Shrike/Kernels/CPU/CPUExpertFFN.swift:102-140 with the generic-bit body), every one over the
    same activation row (the cost of an evaluation does not depend on the row)."""
    from oracle import oracle as O
    off, _ = O.expert_offsets(d, f, bits)
    cores = min(pairs, len(os.sched_getaffinity(0)))
    x = S.SeedTree(0xC0FFEE).key("x").normal(d)
    rng = np.random.default_rng(1)
    weights = np.full(pairs, 1.0 / pairs, np.float32)
    t0 = time.perf_counter()
    for _ in range(evaluations):
        picks = rng.choice(len(blobs), pairs, replace=pairs > len(blobs))
        O.cpu_layer_fp32([blobs[int(e)] for e in picks], weights, off, x, d, f, cores, bits=bits, meta=meta)
    per_step = (time.perf_counter() - t0) / evaluations
    return {"us_per_step": round(per_step * 1e6, 1), "cores": cores, "kind": "port",
            "sample": f"{evaluations} evaluations of {label}, fp32 scalar C port, {cores} threads, gcc -O2"}


def prefill_workload(args, rt, capi, S, meta):
    """Config 3: one ragged prefill chunk of T tokens through router -> grouping -> grouped expert FFN
    -> reduce, top-8 of 256 int4 experts with a Zipf skew injected through the router's logit-bias
    operand. Steps alternate between layers with their own pools so the experts stream from HBM."""
    T = args.tokens
    n_layers = min(args.layers, 3)
    layers, off, stride, keep, gen_s = build_layers(rt, capi, S, n_layers, meta, shared=False)
    moe = rt.MoE(D, F, NE, K, routed_bits=BITS, router_bits=0, meta=meta)
    stream = rt.Stream()
    moe.stream = stream
    pf = rt.Prefill(moe)
    tree = S.SeedTree(0x5EED0003)
    perm = np.argsort(tree.key("zipf.perm").next(NE))
    bias = np.zeros(NE, np.float32)
    bias[perm] = -1.1 * np.log(np.arange(NE) + 1.0)
    d_bias = rt.dev(S.f32_to_bf16_bits(bias))
    ones_d, ones_e = keep[0], keep[1]
    hidden = rt.dev(S.activations_f16(tree, "x", T * D))
    idx, w, logits = rt.empty(4 * T * K), rt.empty(2 * T * K), rt.empty(pf.router_workspace_bytes(T, NE, D))
    routes = rt.GroupedRoutesDevice(T * K, NE)
    partials, h2 = rt.empty(2 * T * K * D), rt.empty(2 * T * D)
    work = rt.empty(pf.ffn_workspace_bytes(T, routes.max_row_tiles))

    # the router's pass over `hidden` also leaves the group sums that the FFN's bias term needs (one launch fewer a chunk);
    # --prefill-two-passes: each of the two reads `hidden` for itself, as the reference's operators do
    fused_sums = not getattr(args, "prefill_two_passes", False)

    def router(lay):
        pf.encode_block(lay["router"], None, None, hidden, ones_d, ones_e, d_bias, idx, w, logits, T, NE, D, K, D,
                        ffn_workspace=work if fused_sums else None)

    def group(lay):
        pf.group_pairs(idx, w, T, K, NE, routes, residency=lay["pool"].table)

    def ffn(lay):
        pf.encode_grouped_expert_gemms(lay["pool"], off, routes, hidden, D, partials, work, T, K, presummed=fused_sums)

    def reduce(lay):
        pf.encode_reduce_token_major(partials, w, h2, T, K, D)

    def step(lay):
        router(lay); group(lay); ffn(lay); reduce(lay)

    def timed(fn, n, regions=1):
        times = []
        stream.synchronize()
        for _ in range(regions):
            start, stop = rt.Event(), rt.Event()
            start.record(stream)
            for i in range(n):
                fn(layers[i % n_layers])
            stop.record(stream)
            stop.synchronize()
            times.append(start.elapsed_ms(stop) / n)
        return statistics.median(times)

    steps, warm = max(6, args.steps // 40), max(3, args.warmup // 40)
    timed(step, warm)
    ms = timed(step, steps, regions=5)
    parts = {name: timed(fn, max(6, steps // 2), regions=3) * 1e3 for name, fn in
             (("router (2 launches)", router), ("grouping (1 launch)", group), ("reduce", reduce))}
    # The FFN's time depends on the routes it is given (the chip holds 512 of its workgroups at a time, and a
    # chunk's row tiles make about that many), so it is timed on each layer's own routes and the middle one is quoted.
    by_layer = []
    for lay in layers:
        router(lay); group(lay)
        # these routes over every layer's pool in turn (an expert sits in the same cell of each), so that the experts
        # come from HBM as in the chunk above and not from the Infinity Cache, which holds one layer's experts whole
        us = timed(ffn, max(6, steps // 2), regions=3) * 1e3
        us_one_pool = timed(lambda _, lay=lay: ffn(lay), max(6, steps // 2), regions=3) * 1e3
        counts = routes.counts.download(np.uint32, NE)
        # the table's eighths (the first tiles mod 8 of them one tile longer): what an XCD takes where the launch does not fit the
        # chip at once; where it does, the kernels even out the tiles of more than 32 rows over the XCDs
        tile_rows = routes.download()["row_tiles"][:, 2]
        q, r = divmod(len(tile_rows), 8)
        starts = [x * q + min(x, r) for x in range(9)]
        by_layer.append({"us": round(us, 2), "us_on_one_pool_over_and_over": round(us_one_pool, 2), "row_tiles": int(routes.row_tile_count.download(np.uint32, 1)[0]),
                         "tiles_by_table_eighth": [starts[x + 1] - starts[x] for x in range(8)],
                         "tiles_over_32_rows_by_table_eighth": [int(np.count_nonzero(tile_rows[starts[x]:starts[x + 1]] > 32)) for x in range(8)],
                         "experts_with_pairs": int(np.count_nonzero(counts)),
                         "mfma_row_tiles_of_32": int(sum((min(64, c - j) + 31) // 32 for c in counts.tolist() for j in range(0, c, 64)))})
    quoted = sorted(by_layer, key=lambda r: r["us"])[len(by_layer) // 2]
    ffn_name = "grouped FFN (2 launches)" if fused_sums else "grouped FFN (3 launches)"
    parts = {"router (2 launches)": parts["router (2 launches)"], "grouping (1 launch)": parts["grouping (1 launch)"],
             ffn_name: quoted["us"], "reduce": parts["reduce"]}
    tiles, used, m_tiles = quoted["row_tiles"], quoted["experts_with_pairs"], quoted["mfma_row_tiles_of_32"]
    expert_bytes = used * stride
    algorithmic = expert_bytes + 2 * T * D * 2 + T * K * 16
    flops = T * K * 6 * D * F
    ffn_us = parts[ffn_name]
    traffic = profile_figure("prefill_chunk_q35b_int4_t512.txt", "hbm_bytes_per_chunk_grouped_ffn") if T == 512 else None
    # What a SIMD makes of matrix and vector instructions side by side, at the FFN kernels' two waves a SIMD: a slot of
    # four 32x32x16 matrix instructions, a slot of thirty-two fused multiply-adds, and both (the FFN's main loop issues
    # about as many cycles of each). Where `both` is near the sum and not near the longer one, the kernel's floor is
    # the sum of its matrix and vector cycles, not the larger.
    from harness import probes
    one, sink = rt.dev(np.ones(1, np.float32)), rt.empty(64)
    slots = 2048

    def issue_us(what, waves):
        def fn(_):
            probes.check(probes.load().shrike_probe_issue(stream.handle, what, waves, slots, one.ptr, sink.ptr), "probe_issue")
        return timed(fn, 4, regions=3) * 1e3
    issue = {"slots": slots, "slot": "4 x v_mfma_f32_32x32x16_f16 | 32 x v_fma_f32", "by_waves_per_simd": {}}
    for waves in (2, 4):
        m_us, v_us, b_us = issue_us(1, waves), issue_us(2, waves), issue_us(3, waves)
        issue["by_waves_per_simd"][str(waves)] = {"matrix_us": round(m_us, 1), "vector_us": round(v_us, 1), "both_us": round(b_us, 1),
                                                 "both_over_longer": round(b_us / max(m_us, v_us), 3),
                                                 "both_over_sum": round(b_us / (m_us + v_us), 3)}
    cpu = None
    if getattr(args, "cpu_sample", 0) > 0:  # the chunk's T * K pair FFNs on the host's cores
        cpu = cpu_pairs(S, keep[4], D, F, BITS, meta, T * K, 1, f"one chunk's {T * K} pair FFNs at the 35B-A3B shape, int4")
        cpu["us_per_chunk"] = cpu.pop("us_per_step")
    return {
        **({"cpu_baseline": cpu} if cpu else {}),
        "metric": "ragged prefill chunk through the routed experts: tokens/s (ms per chunk in ms_per_step), 35B-A3B int4 shape",
        "value": round(T / (ms * 1e-3), 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warm,
        "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16 x u4 -> f32",
        "data": "synthetic (seeded SplitMix64: uniform int4 codes, |N(0,0.02)| scales, N(0,1) fp16 activations, Zipf(1.1) expert skew)",
        "config": {"workload": f"config 3: ragged prefill, {T} tokens, top-8 of 256 int4 experts (hidden 2048, intermediate 512), "
                               "router + device grouping + grouped FFN + reduce, all slots resident",
                   "stacked_layers": n_layers, "meta_dtype": args.meta, "experts_with_pairs": used, "row_tiles": tiles,
                   "mfma_row_tiles_of_32": m_tiles,
                   "hidden_group_sums": "left by the router's select launch (shrike_hip_prefill_router_with_group_sums + "
                                        "shrike_hip_prefill_grouped_ffn_presummed)" if fused_sums else
                                        "formed by the grouped FFN's own first launch (the two-pass entry points)"},
        "kernel_us_per_chunk": {k: round(v, 2) for k, v in parts.items()},
        "grouped_ffn_by_layer_routes": by_layer,
        "roofline": {"bound": "hbm", "kernel": "k_grouped_ffn<4,0> + k_grouped_ffn<4,1> (gate/up + down of every row tile)",
                     "achieved": round(expert_bytes / (ffn_us * 1e-6) / 1e9, 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(expert_bytes / (ffn_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4), "bytes_per_launch": expert_bytes,
                     "us_per_launch": round(ffn_us, 2), "traffic": traffic,
                     "mfma_tflops_on_pair_flops": round(flops / (ffn_us * 1e-6) / 1e12, 2),
                     "matrix_and_vector_issue": issue},
        "algorithmic_bytes_per_chunk": algorithmic, "pair_flops_per_chunk": flops,
    }


def gptoss_workload(args, rt, capi, S, meta, bits):
    """Config 4: a batch of 4 independent tokens through 24 stacked gpt-oss-20B-shape layers (hidden 2880,
    32 experts of intermediate 2880, top-4, int4 or int8 codes): router -> resolve -> phase 1 -> phase 2 with the
    token dimension on the grid, every layer with its own pool."""
    d = f = 2880
    ne, k, t, n_layers = 32, 4, 4, min(args.layers, 24)
    tree = S.SeedTree(0x5EED0004)
    off, stride = rt.expert_offsets(d, f, bits)
    blobs = [S.expert_blob(tree, f"layer.0.expert.{e}", d, f, bits, meta) for e in range(ne)]
    pools, routers = [], []
    for l in range(n_layers):
        pool = rt.ExpertPool(ne, stride, ne)
        if l == 0:
            for e in range(ne):
                capi.check(capi.load().shrike_hip_memcpy_h2d(pool.cell_ptr(e), blobs[e].ctypes.data, blobs[e].nbytes), "h2d")
        else:
            capi.check(capi.load().shrike_hip_memcpy_d2d(pool.cell_ptr(0), pools[0].cell_ptr(0), ne * pool.stride), "d2d")
        for e in range(ne):
            pool.publish(e, e, capi.RESIDENT)
        pools.append(pool)
        routers.append(rt.dev(S.router_f16(tree, f"layer.{l}.router.w", ne, d)))
    cpu = None
    if getattr(args, "cpu_sample", 0) > 0:  # one layer's 16 (token, expert) FFNs on the host's cores
        cpu = cpu_pairs(S, blobs, d, f, bits, meta, t * k, 3, f"one layer's {t * k} expert FFNs at the gpt-oss shape, int{bits}")
        cpu["us_per_layer"] = cpu.pop("us_per_step")
    del blobs
    moe = rt.MoE(d, f, ne, k, routed_bits=bits, router_bits=0, meta=meta)
    stream = rt.Stream()
    moe.stream = stream
    pf = rt.Prefill(moe)
    ones_d, ones_e = rt.dev(S.f32_to_bf16_bits(np.ones(d, np.float32))), rt.dev(S.f32_to_bf16_bits(np.ones(ne, np.float32)))
    zeros_e = rt.dev(np.zeros(ne, np.uint16))
    hidden = rt.dev(S.activations_f16(tree, "x", t * d))
    idx, w, rws = rt.empty(4 * t * k), rt.empty(2 * t * k), rt.empty(pf.router_workspace_bytes(t, ne, d))
    routes = rt.GroupedRoutesDevice(t * k, ne)
    partials, h2 = rt.empty(2 * t * k * d), rt.empty(2 * t * d)
    work = rt.empty(pf.ffn_workspace_bytes(t, routes.max_row_tiles))

    resolved, acts, y = rt.empty(4 * t * k), rt.empty(2 * t * k * f), rt.empty(2 * t * d)
    # diagnostics: the prefill operators instead of the decode ones; the decode operators one by one (router, resolve,
    # phase 1, phase 2: four launches) instead of the fused layer for a batch (three)
    grouped = os.environ.get("SHRIKE_BENCH_GROUPED") == "1"
    split = os.environ.get("SHRIKE_BENCH_SPLIT") == "1"
    layer_args = []
    for l in range(n_layers):
        a = capi.DecodeLayerArgs()
        a.router_weights, a.effective_scale, a.per_expert_scale, a.logit_bias = routers[l].ptr, ones_d.ptr, ones_e.ptr, zeros_e.ptr
        a.pool, a.pool_slot_stride, a.residency, a.offsets = pools[l].bases, pools[l].stride, pools[l].table, off
        a.x, a.y, a.out_indices, a.out_weights, a.resolved_slots, a.acts = hidden.ptr, y.ptr, idx.ptr, w.ptr, resolved.ptr, acts.ptr
        layer_args.append(a)

    def all_layers():
        for l in range(n_layers):
            if not grouped and not split:
                moe.encode_decode_layer_batch(layer_args[l], t, d)
                continue
            pf.encode_block(routers[l], None, None, hidden, ones_d, ones_e, zeros_e, idx, w, rws, t, ne, d, k, d)
            if grouped:
                pf.group_pairs(idx, w, t, k, ne, routes, residency=pools[l].table)
                pf.encode_grouped_expert_gemms(pools[l], off, routes, hidden, d, partials, work, t, k)
                pf.encode_reduce_token_major(partials, w, h2, t, k, d)
            else:
                moe.encode_resolve_batch(idx, pools[l].table, resolved, t * k, ne)
                moe.encode_phase1_batch(pools[l], resolved, off, hidden, d, acts, d, f, k, t)
                moe.encode_phase2_batch(pools[l], resolved, off, acts, w, None, y, None, d, f, k, t)

    all_layers()
    stream.synchronize()
    graph = capture(rt, capi, stream, all_layers)
    reps = max(2, args.steps // 200)
    time_graph(rt, capi, stream, graph, max(1, args.warmup // 200))
    ms = median_of_regions(rt, capi, stream, graph, reps, regions=7)
    # distinct experts differ per layer (own router); count them from one eager pass per layer
    distinct = []
    for l in range(n_layers):
        pf.encode_block(routers[l], None, None, hidden, ones_d, ones_e, zeros_e, idx, w, rws, t, ne, d, k, d)
        stream.synchronize()
        distinct.append(len(set(idx.download(np.uint32, t * k).tolist())))
    expert_bytes = sum(distinct) * stride
    capi.check(capi.load().shrike_hip_graph_destroy(graph), "graph_destroy")
    return {
        "metric": "gpt-oss-20B-shape MoE layers, 4 tokens: us per layer (ms per 24-layer stack in ms_per_step)",
        "value": round(expert_bytes / (ms * 1e-3) / 1e9, 2), "unit": "GB/s", "n_gpus": 1, "steps": reps, "warmup": max(1, args.warmup // 200),
        "ms_per_step": round(ms, 5), "us_per_layer": round(ms * 1e3 / n_layers, 2), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16 x u%d -> f32" % bits, "data": "synthetic (seeded SplitMix64)",
        "config": {"workload": f"config 4: {t} tokens, top-{k} of {ne} int{bits} experts, hidden {d}, intermediate {f}, {n_layers} stacked layers "
                               "in one HIP graph, all slots resident",
                   "operators": "grouped (prefill)" if grouped else "batched decode, four operators a layer" if split else
                                "the fused layer for a batch (three launches a layer)",
                   "distinct_experts_per_layer": distinct, "expert_bytes_per_stack": expert_bytes,
                   "pair_bytes_per_stack": n_layers * t * k * stride, "meta_dtype": args.meta},
        "GBps_on_pair_bytes": round(n_layers * t * k * stride / (ms * 1e-3) / 1e9, 2),
        "hbm_peak_frac_on_expert_bytes": round(expert_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
        **({"cpu_baseline": cpu} if cpu else {})}


def kimi_workload(args, rt, capi, S, meta):
    """Config 5: 16 sequences, one token each, Kimi-Linear-48B shape (hidden 2304, 256 int8 experts of
    intermediate 1024, top-8, shared expert 1024); the pool holds 64 of the 256 experts and misses are copied
    from pinned host memory on a side stream. Reports the miss rate, the wall time per step and the host->device
    rate; beside them the step with every expert resident (what the kernels alone take), the step's time on each
    stream (how much of the copies runs beside kernels), and the miss rate under the other eviction policy."""
    from harness import runners
    from shrike_amd import host as HL
    d, f, ne, k, t, bits, slots = 2304, 1024, 256, 8, 16, 8, 64
    tree = S.SeedTree(0x5EED0005)
    off, stride = rt.expert_offsets(d, f, bits)
    store = rt.PinnedBuffer(ne * stride)
    for e in range(ne):
        store.array[e * stride:(e + 1) * stride] = S.expert_blob(tree, f"layer.0.expert.{e}", d, f, bits, meta)
    moe = rt.MoE(d, f, ne, k, routed_bits=bits, router_bits=0, meta=meta)
    moe.stream = rt.Stream()
    router = dict(weights=rt.dev(S.router_f16(tree, "router.w", ne, d)), eff_scale=rt.dev(S.f32_to_bf16_bits(np.ones(d, np.float32))),
                  expert_scale=rt.dev(S.f32_to_bf16_bits(np.ones(ne, np.float32))), bias=rt.dev(np.zeros(ne, np.uint16)))
    shared = {n: tuple(rt.dev(a) for a in S.affine_matrix(tree.key(f"shared.{n}"), r, c, bits, meta))
              for n, r, c in (("gate", f, d), ("up", f, d), ("down", d, f))}
    h1 = rt.empty(2 * t * d)
    batches = [rt.dev(S.activations_f16(tree, f"x.{i}", t * d)) for i in range(8)]
    steps, warm = max(8, args.steps // 100), 8

    def run(cells, slru_share, steps, trace=False):
        """`steps` steps through a pool of `cells` cells under one eviction policy, after 8 warm-up steps."""
        pool = rt.ExpertPool(cells, stride, ne)
        cache = HL.SlotCache(cells, ne, slru_share=slru_share)
        layer = runners.BatchedDecodeLayer(moe, pool, cache, off, store, stride, stride, t)
        sws = [None]

        def step(i):
            x = batches[i % len(batches)]
            layer.run(router, x, t, d)

            def tail():
                sws[0] = layer.pf.encode_shared_expert(shared["gate"], shared["up"], shared["down"], bits, x, d, h1, t, f, workspace=sws[0])
                layer.pf.residual_add(layer.h2, h1, t * d)
            if layer.trace is None:
                tail()
            else:
                start, stop = rt.Event(), rt.Event()
                start.record(moe.stream)
                tail()
                stop.record(moe.stream)
                layer.trace.append(("compute", start, stop))
            moe.stream.synchronize()

        for i in range(warm):
            step(i)
        base = cache.statistics(stride)
        base = (base.requested_experts, base.misses, base.bytes_read, base.plans)
        if trace:
            layer.trace = []
        t0 = time.perf_counter()
        for i in range(steps):
            step(warm + i)
        dt = time.perf_counter() - t0
        st = cache.statistics(stride)
        out = dict(dt=dt, steps=steps, requested=st.requested_experts - base[0], misses=st.misses - base[1],
                   read=st.bytes_read - base[2], plans=st.plans - base[3], on_stream={})
        if trace:
            for name, start, stop in layer.trace:
                out["on_stream"][name] = out["on_stream"].get(name, 0.0) + start.elapsed_ms(stop)
        pool.close()
        return out

    main = run(slots, None, steps)
    dt, req, miss, read, plans = main["dt"], main["requested"], main["misses"], main["read"], main["plans"]
    # the same steps with every expert resident (256 cells): what the kernels alone take, every route a hit
    resident = run(ne, None, steps)
    # the step's time on each stream (events round everything enqueued), a shorter run of its own: kernels and copies
    # summed apart against the wall clock say how much of one runs beside the other
    traced = run(slots, None, max(4, steps // 4), trace=True)
    n_tr = traced["steps"]
    copy_ms, kernel_ms, wall_ms = traced["on_stream"].get("upload", 0.0) / n_tr, traced["on_stream"].get("compute", 0.0) / n_tr, traced["dt"] / n_tr * 1e3
    slru = run(slots, 0.5, max(8, steps // 2))
    cpu = None
    if getattr(args, "cpu_sample", 0) > 0:  # one step's 128 routed + 16 shared-expert FFNs on the host's cores
        views = [store.array[e * stride:e * stride + stride] for e in range(0, ne, 4)]
        cpu = cpu_pairs(S, views, d, f, bits, meta, t * k + t, 2, f"one step's {t * k} routed and {t} shared-expert FFNs at the Kimi shape, int8")
    return {
        "metric": "Kimi-Linear-48B-shape MoE decode, 16 sequences through a 64-of-256 slot pool: ms per step (wall clock, misses included)",
        "value": round(t / (dt / steps), 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warm,
        "ms_per_step": round(dt / steps * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 x u8 -> f32", "data": "synthetic (seeded SplitMix64), 8 token batches in rotation",
        "config": {"workload": f"config 5: {t} sequences, top-{k} of {ne} int8 experts, hidden {d}, intermediate {f}, shared expert {f}, "
                               f"pool of {slots} cells, misses from pinned host memory on a side stream",
                   "passes_per_step": round(plans / steps, 2), "eviction": "aging LFU (the reference's default)"},
        "miss_rate": round(miss / max(1, req), 4), "experts_requested_per_step": round(req / steps, 1),
        "host_to_device_GBps": round(read / dt / 1e9, 2), "bytes_copied_per_step": int(read / steps),
        "hit_only_kernel_ms": round(resident["dt"] / resident["steps"] * 1e3, 4),
        "hit_only": {"cells": ne, "miss_rate": round(resident["misses"] / max(1, resident["requested"]), 4),
                     "note": "the same steps through a pool that holds all 256 experts: router, grouping, grouped FFN, reduce, shared "
                             "expert, wall clock with the step's host synchronisations"},
        "timeline_ms_per_step": {"copies_on_the_upload_stream": round(copy_ms, 4), "kernels_on_the_compute_stream": round(kernel_ms, 4),
                                 "wall_clock": round(wall_ms, 4)},
        "copy_ms_hidden_behind_compute": round(max(0.0, copy_ms + kernel_ms - wall_ms), 4),
        "miss_rate_by_policy": {"aging_lfu": round(miss / max(1, req), 4),
                                "slru_protected_share_0.5": round(slru["misses"] / max(1, slru["requested"]), 4)},
        "miss_rate_floor": round(max(0.0, req / steps - slots) / max(1e-9, req / steps), 4),
        **({"cpu_baseline": cpu} if cpu else {})}


def decode_workload(args, rt, capi, S, meta):
    from harness import probes
    n_layers = args.layers
    layers, off, stride, keep, gen_s = build_layers(rt, capi, S, n_layers, meta, shared=not args.no_shared)
    moe = rt.MoE(D, F, NE, K, routed_bits=BITS, router_bits=0, meta=meta)
    stream = rt.Stream()
    moe.stream = stream

    def all_layers():
        for lay in layers:
            moe.encode_decode_layer(lay["args"])

    all_layers()  # eager pass: fills every layer's routing scratch
    stream.synchronize()

    # ---- the headline: exactly K steps a region, REGIONS regions, median
    steps, warm = max(1, args.steps), max(0, args.warmup)
    walk = LayerWalk(rt, capi, moe, stream, layers)
    walk.plan(warm, 1)
    walk.enqueue(warm)
    region_ms, timing_method, whole_graph_us, empty_region_us = None, None, None, None
    from harness import probes as _probes
    clock_khz = _probes.load().shrike_probe_wall_clock_khz()
    if args.timing == "graph" and clock_khz > 0:
        # All REGIONS regions are ONE captured graph with a time-stamp kernel between regions (one thread stores the
        # device's constant-rate clock, in graph order): a region is then K layers and one 64-thread launch, where a
        # graph launch per region bills every region a launch boundary of its own (about 19 us on this part, which a
        # 20-layer region feels). HIP events cannot do this: an event recorded by a captured graph cannot be timed
        # (hipEventElapsedTime: invalid resource handle). Events still bracket the whole graph as the cross-check.
        # One more stamp follows the last region's at once: the two bracket nothing, which is what a region holds besides
        # its K layers (reported as "empty_region_us", not subtracted).
        stamps = rt.empty(8 * (REGIONS + 2)).fill(0)

        def regions_body():
            _probes.check(_probes.load().shrike_probe_timestamp(stream.handle, stamps.ptr), "probe_timestamp")
            for r in range(REGIONS):
                walk.encode(steps)
                _probes.check(_probes.load().shrike_probe_timestamp(stream.handle, stamps.ptr + 8 * (r + 1)), "probe_timestamp")
            _probes.check(_probes.load().shrike_probe_timestamp(stream.handle, stamps.ptr + 8 * (REGIONS + 1)), "probe_timestamp")
        timed = capture(rt, capi, stream, regions_body)
        first, last = rt.Event(), rt.Event()
        stream.synchronize()
        rt.synchronize()
        first.record(stream)
        capi.check(capi.load().shrike_hip_graph_launch(timed, stream.handle), "graph_launch")
        last.record(stream)
        last.synchronize()
        rt.synchronize()
        ticks = stamps.download(np.uint64, REGIONS + 2).astype(np.int64)
        region_ms = [float(ticks[r + 1] - ticks[r]) / clock_khz for r in range(REGIONS)]
        empty_region_us = float(ticks[REGIONS + 1] - ticks[REGIONS]) / clock_khz * 1e3
        whole_graph_us = first.elapsed_ms(last) * 1e3 / (REGIONS * steps)
        capi.check(capi.load().shrike_hip_graph_destroy(timed), "graph_destroy")
        timing_method = (f"one captured graph of {REGIONS} regions of K layers, the device clock ({clock_khz} kHz) stored by a "
                         "one-thread kernel between regions; HIP events round the whole graph as the cross-check")
    if region_ms is None:
        events = [rt.Event() for _ in range(REGIONS + 1)]
        walk.plan(steps, REGIONS)
        stream.synchronize()
        rt.synchronize()
        events[0].record(stream)
        for r in range(REGIONS):
            walk.enqueue(steps)
            events[r + 1].record(stream)
        events[-1].synchronize()
        rt.synchronize()
        region_ms = [events[r].elapsed_ms(events[r + 1]) for r in range(REGIONS)]
        timing_method = "graph launches of up to 40 layers, a HIP event record between regions"
    ms_per_step = statistics.median(region_ms) / steps
    # the experts a pass over the stack touches, per activation variant (routes differ from variant to variant)
    distinct = set()
    for v in range(X_VARIANTS):
        for l, lay in enumerate(layers):
            moe.encode_decode_layer_launches(lay["args_x"][v], 3)
            stream.synchronize()
            distinct.update((l, int(e)) for e in lay["idx"].download(np.uint32, K))

    # ---- the layer's launches one at a time (each in a graph of its own over the whole stack), the split operators
    # and the two floors, for the per-kernel figures
    def launches(mask):
        def body():
            for lay in layers:
                moe.encode_decode_layer_launches(lay["args"], mask)
        return body

    def phase1_only():
        for lay in layers:
            moe.encode_spec_phase1(lay["pool"], lay["res"], off, lay["x"], lay["acts"], D, F, K)

    def phase2_only():
        for lay in layers:
            moe.encode_spec_phase2(lay["pool"], lay["res"], off, lay["acts"], lay["w"], lay["h1"], lay["y"], None, D, F, K)

    def router_only():
        for lay in layers:
            a = lay["args"]
            moe.encode_router(a.router_weights, None, None, a.x, a.effective_scale, a.per_expert_scale, a.logit_bias,
                              a.out_indices, a.out_weights, NE, D, K)

    def shared_only():
        for lay in layers:
            sh = lay["shared"]
            moe.encode_shared_expert(sh["gate"], sh["up"], sh["down"], BITS, lay["x"], lay["ss"], lay["h1"], D, FS)

    # the floors a launch is bounded by on this part: a launch with nothing to do, and a kernel that only
    # reads the bytes phase 1 reads (gate + up sub-tensors of the same eight cells) with no arithmetic
    sink = rt.empty(4)
    p1_blocks = K * F // 4 // 4
    p1_bytes_per_cell = 2 * (F * D // 2 + 2 * F * (D // 64) * 2)

    def empty_only():
        for lay in layers:
            probes.check(probes.load().shrike_probe_empty_launch(stream.handle, p1_blocks, sink.ptr), "probe_empty_launch")

    def read_only():
        for lay in layers:
            probes.check(probes.load().shrike_probe_read(stream.handle, lay["pool"].bases, lay["pool"].stride, lay["res"].ptr,
                                                         K, off.gate_w_off, p1_bytes_per_cell, sink.ptr), "probe_read")

    # a memory round trip as a kernel sees it: one wave walks CHASE_HOPS dependent loads through a 128 MB table, 4 MB and
    # a line apart (every hop a miss of the caches on the compute units' side); each launch starts elsewhere
    chase_words, chase_stride = 32 << 20, (1 << 20) + 16
    chase = rt.dev(((np.arange(chase_words, dtype=np.uint64) + chase_stride) % chase_words).astype(np.uint32))

    def empty_one():
        for lay in layers:
            probes.check(probes.load().shrike_probe_empty_launch(stream.handle, 1, sink.ptr), "probe_empty_launch")

    def chase_only():
        for l, lay in enumerate(layers):
            probes.check(probes.load().shrike_probe_dependent_loads(stream.handle, chase.ptr, chase_words, CHASE_HOPS, 4099 * l + 64,
                                                                    sink.ptr), "probe_dependent_loads")

    # the step ahead of the layer (residual add + RMS norm producing x): as a launch of its own, and in the
    # prologue of the layer's first launch; both on a residual stream and an x buffer of their own
    tree_n = S.SeedTree(0x5EED0003)
    hidden_n, x_n = rt.dev(S.activations_f16(tree_n, "hidden", D)), rt.empty(2 * D)
    delta_n = rt.dev(S.f32_to_f16_bits(tree_n.key("delta").normal(D, std=0.05)))
    weight_n = rt.dev(S.f32_to_bf16_bits(tree_n.key("weight").uniform(0.5, 1.5, D)))
    normed_args = []
    for lay in layers:
        apart_a, fused_a = capi.DecodeLayerArgs(), capi.DecodeLayerArgs()
        for dst in (apart_a, fused_a):
            C.memmove(C.byref(dst), C.byref(lay["args"]), C.sizeof(dst))
            dst.x, dst.hidden = x_n.ptr, hidden_n.ptr
        fused_a.norm_delta, fused_a.norm_weight, fused_a.norm_eps = delta_n.ptr, weight_n.ptr, 1e-6
        normed_args.append((apart_a, fused_a))

    def norm_apart():
        for apart_a, _ in normed_args:
            rt.residual_add_rmsnorm_bf16w(hidden_n, delta_n, weight_n, x_n, D, 1e-6, 1, stream=stream)
            moe.encode_decode_layer(apart_a)

    def norm_fused():
        for _, fused_a in normed_args:
            moe.encode_decode_layer(fused_a)

    reps = max(2, min(10, steps // n_layers))
    parts = {}
    for name, body in (("launch 1: router rows + route entries + shared gate/up rows (k_head)", launches(1)),
                       ("launch 2: select + routed gate/up rows + shared down rows (k_phase1, routing)", launches(2)),
                       ("launch 3: routed down rows + combine (k_phase2)", launches(4)),
                       ("operator: phase 1 alone (no routing, no shared rows)", phase1_only),
                       ("operator: phase 2 alone", phase2_only),
                       ("operator: router + select + classify", router_only),
                       ("operator: shared expert (2 launches)", shared_only),
                       ("floor: empty launch of phase 1's grid", empty_only),
                       ("floor: read-only kernel over phase 1's routed bytes", read_only),
                       ("floor: empty launch of one workgroup", empty_one),
                       (f"floor: one wave, {CHASE_HOPS} dependent loads", chase_only),
                       ("norm launch + layer (4 launches)", norm_apart),
                       ("layer with the norm in its first launch", norm_fused)):
        g = capture(rt, capi, stream, body)
        time_graph(rt, capi, stream, g, 2)
        parts[name] = median_of_regions(rt, capi, stream, g, reps, regions=7) / n_layers * 1e3  # us per layer
        capi.check(capi.load().shrike_hip_graph_destroy(g), "graph_destroy")

    expert_bytes = (K + 1) * stride  # 15,925,248
    total_bytes = expert_bytes + NE * D * 2 + 2 * D * 2
    routed_gate_up = K * 2 * (F * D // 2 + 2 * F * (D // 64) * 2)      # gate+up codes, scales and biases of 8 experts
    shared_down = D * FS // 2 + 2 * D * (FS // 64) * 2                  # the shared expert's down rows ride in launch 2
    launch2_bytes = routed_gate_up + (0 if args.no_shared else shared_down)
    launch2_us = parts["launch 2: select + routed gate/up rows + shared down rows (k_phase1, routing)"]
    alone_us = parts["operator: phase 1 alone (no routing, no shared rows)"]
    value = expert_bytes / (ms_per_step * 1e-3) / 1e9
    meta_param = 1 if args.meta == "f16" else 0  # the kernels' last template parameter: SHRIKE_META_F16 = 1, SHRIKE_META_BF16 = 0
    kernel = f"k_phase1<4,1,4,true,4,true,false,{meta_param}>"
    # The floor of the layer AS IT IS BUILT (three launches in a row, five dependent memory round trips: x and rows in
    # the first; the route table, then rows in the second; cells and activations, then rows in the third), from this
    # run's own probes: launches x an empty launch + round trips x one dependent load + the layer's bytes at the rate
    # the read-only kernel streams at once it has started.
    empty_us = parts["floor: empty launch of phase 1's grid"]
    read_us = parts["floor: read-only kernel over phase 1's routed bytes"]
    hop_us = max(0.0, parts[f"floor: one wave, {CHASE_HOPS} dependent loads"] - parts["floor: empty launch of one workgroup"]) / CHASE_HOPS
    stream_gbps = routed_gate_up / max(1e-9, (read_us - empty_us) * 1e-6) / 1e9
    floor_us = 3 * empty_us + 5 * hop_us + total_bytes / (stream_gbps * 1e9) * 1e6
    out = {
        "metric": "MoE-layer decode: HBM GB/s on expert bytes (us per layer in ms_per_step), 35B-A3B int4 shape",
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": steps, "warmup": warm,
        "ms_per_step": round(ms_per_step, 6), "us_per_layer": round(ms_per_step * 1e3, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic (seeded SplitMix64: uniform int4 codes, |N(0,0.02)| scales, N(0,1) fp16 activations)",
        "config": {"workload": "config 2: full MoE layer decode, 1 token, hidden 2048, top-8 of 256 int4 experts "
                               "(intermediate 512, group 64) + 1 shared expert, fp16 router, all slots resident",
                   "stacked_layers": n_layers, "pool_bytes_total": n_layers * NE * stride,
                   "pools": "layer 0's experts come from the seeded generator; layers 1.. hold byte copies of layer 0's pool at "
                            "addresses of their own (routers, shared experts and activations are distinct per layer)",
                   "activation_variants": X_VARIANTS,
                   "expert_bytes_touched_by_a_pass_over_every_variant": len(distinct) * stride,
                   "meta_dtype": args.meta, "launches_per_layer": 3, "hip_graph": True},
        "timing": {"regions": REGIONS, "steps_per_region": steps, "statistic": "median", "method": timing_method,
                   "us_per_layer_min": round(min(region_ms) / steps * 1e3, 3),
                   "us_per_layer_max": round(max(region_ms) / steps * 1e3, 3),
                   **({"us_per_layer_by_hip_events_round_all_regions": round(whole_graph_us, 3)} if whole_graph_us else {}),
                   **({"empty_region_us": round(empty_region_us, 3)} if empty_region_us is not None else {})},
        "hbm_peak_frac_on_expert_bytes": round(value / HBM_PEAK_GBPS, 4),
        "expert_bytes_per_step": expert_bytes, "total_bytes_per_step": total_bytes,
        "kernel_us_per_layer": {k: round(v, 3) for k, v in parts.items()},
        "roofline": {"bound": "hbm", "kernel": kernel + " (the layer's second launch: every wave selects from the route entries, "
                                               "routed gate/up matvec + SiLU-multiply, shared expert's down rows)",
                     "achieved": round(launch2_bytes / (launch2_us * 1e-6) / 1e9, 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(launch2_bytes / (launch2_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                     "bytes_per_launch": launch2_bytes, "us_per_launch": round(launch2_us, 3),
                     "traffic": profile_figure("decode_phase1_q35b_int4_hbm_traffic.txt", "hbm_bytes_per_launch"),
                     "standalone_operator": {"kernel": f"k_phase1<4,1,2,false,0,true,false,{meta_param}> (gate/up rows alone: no routing, two row pairs a wave)", "bytes_per_launch": routed_gate_up,
                                             "us_per_launch": round(alone_us, 3),
                                             "frac": round(routed_gate_up / (alone_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)},
                     "traffic_source": "profiles/decode_phase1_q35b_int4_hbm_traffic.txt (FETCH_SIZE + WRITE_SIZE of a profiled run "
                                       "of this kernel, scaled by a copy's; not measured by this run)",
                     "floors_us": {"empty_launch": round(empty_us, 3), "read_only_same_bytes": round(read_us, 3)},
                     "design_floor_us": round(floor_us, 2),
                     "design_floor": {"launches": 3, "empty_launch_us": round(empty_us, 3), "dependent_round_trips": 5,
                                      "round_trip_us": round(hop_us, 3), "bytes": total_bytes,
                                      "streamed_GBps": round(stream_gbps, 1),
                                      "frac_of_peak_at_the_floor": round(expert_bytes / (floor_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                                      "measured_over_floor": round(ms_per_step * 1e3 / floor_us, 3)}},
        "setup_seconds": round(gen_s, 1),
    }
    if args.cpu_sample > 0:
        out["cpu_baseline"] = cpu_baseline(S, keep[4], args.cpu_sample, meta)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400, help="layer decodes per timed region (the run times 15 regions)")
    ap.add_argument("--warmup", type=int, default=80)
    ap.add_argument("--layers", type=int, default=40, help="stacked layers with their own pools (40 x 453 MB)")
    ap.add_argument("--meta", choices=["f16", "bf16"], default="f16")
    ap.add_argument("--cpu-sample", type=int, default=3000, help="layer evaluations timed on the CPU, about ten seconds of host work (0 = skip)")
    ap.add_argument("--no-shared", action="store_true", help="diagnostic: leave the shared expert out of the layer")
    ap.add_argument("--no-secondary", action="store_true", help="the headline workload alone")
    ap.add_argument("--timing", choices=["graph", "launches"], default="graph",
                    help="decode: the timed regions in one captured graph with a time-stamp kernel between them (default), or a "
                         "graph launch of up to 40 layers at a time with HIP event records between regions")
    ap.add_argument("--workload", choices=["decode", "prefill", "gptoss", "kimi"], default="decode",
                    help="decode: the headline metric (config 2) with the other workloads in its `secondary` block; "
                         "prefill: the ragged 512-token chunk (config 3) alone; gptoss: 4 tokens through 24 gpt-oss-shape "
                         "layers (config 4) alone; kimi: 16 sequences through a 64-cell pool fed from pinned host memory "
                         "(config 5) alone")
    ap.add_argument("--bits", type=int, choices=[4, 8], default=4, help="gptoss: code width")
    ap.add_argument("--tokens", type=int, default=512, help="prefill: tokens in the chunk")
    ap.add_argument("--prefill-two-passes", action="store_true",
                    help="prefill diagnostic: the router and the grouped FFN each read the hidden rows for themselves")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path is built and measured on a single MI355X "
              "(--gpus N with N > 1 is not supported)", file=sys.stderr)
        sys.exit(2)

    if profiler_attached() and args.steps > PROFILED_MAX_STEPS:
        print(f"bench.py: a profiler is attached and --steps {args.steps} exceeds {PROFILED_MAX_STEPS}, the largest region that has "
              "run clean under rocprofv3 (a profiled run at --steps 2000 once aborted inside hipGraphLaunch and its cause was "
              "never shown); profile at --steps <= 400", file=sys.stderr)
        sys.exit(2)

    from shrike_amd import capi, runtime as rt
    from shrike_amd import synth as S

    rt.init(0)
    meta = S.META_F16 if args.meta == "f16" else S.META_BF16
    if args.workload == "prefill":
        return print(json.dumps(prefill_workload(args, rt, capi, S, meta)))
    if args.workload == "gptoss":
        return print(json.dumps(gptoss_workload(args, rt, capi, S, meta, args.bits)))
    if args.workload == "kimi":
        return print(json.dumps(kimi_workload(args, rt, capi, S, meta)))
    out = decode_workload(args, rt, capi, S, meta)
    if not args.no_secondary:
        # the other workloads of the benchmark definition, measured by this same run with sizes of their own
        side = argparse.Namespace(**vars(args))
        side.steps, side.warmup, side.layers = 4000, 400, 40
        secondary = {}
        for name, run in (("config3_ragged_prefill_512_tokens", lambda: prefill_workload(side, rt, capi, S, meta)),
                          ("config4_gpt_oss_shape_4_tokens_int4", lambda: gptoss_workload(side, rt, capi, S, meta, 4)),
                          ("config4_gpt_oss_shape_4_tokens_int8", lambda: gptoss_workload(side, rt, capi, S, meta, 8)),
                          ("config5_kimi_shape_16_sequences_64_of_256_cells", lambda: kimi_workload(side, rt, capi, S, meta))):
            gc.collect()
            r = run()
            secondary[name] = {k: r[k] for k in r if k in ("metric", "value", "unit", "ms_per_step", "us_per_layer", "config",
                                                           "kernel_us_per_chunk", "grouped_ffn_by_layer_routes", "roofline", "GBps_on_pair_bytes",
                                                           "hbm_peak_frac_on_expert_bytes", "miss_rate", "host_to_device_GBps", "hit_only_kernel_ms", "hit_only",
                                                           "timeline_ms_per_step", "copy_ms_hidden_behind_compute", "miss_rate_by_policy", "miss_rate_floor",
                                                           "bytes_copied_per_step", "experts_requested_per_step", "steps", "dtype", "cpu_baseline")}
        out["secondary"] = secondary
    print(json.dumps(out))


if __name__ == "__main__":
    main()
