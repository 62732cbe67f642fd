"""Runner stand-ins over the operator mirror: the loops a host runs AROUND the operators (the reference's
RealForwardRunner and its tile driver), as the GPU tests and the benchmark need them to drive the library the
way the reference's runner would. They sequence calls into libshrikehip and compute nothing; a host that links
the library brings its own runner, so none of this is part of the product package."""
from __future__ import annotations

import numpy as np

from shrike_amd import capi
from shrike_amd import host as _host
from shrike_amd.capi import SENTINEL, ShrikeError, check
from shrike_amd.runtime import (Event, ExpertPool, GroupedRoutesDevice, MoE, PinnedBuffer, Prefill, Stream, empty,
                                synchronize)

READBACK_POLL_NANOS = 200_000_000  # how long a runner polls the tagged words before it falls back to a synchronise


def read_router_readback(readback: PinnedBuffer, top_k: int, tag: int, compute):
    """The runner's host readback (RealForwardRunner.swift:3294-3310): poll the classifier's tagged words in pinned
    memory while the command still runs; if they do not turn up in time, wait for the stream and decode once more."""
    rb = _host.RouterHostReadback.poll(readback.ptr, top_k, tag, READBACK_POLL_NANOS)
    if rb is None:
        (compute.synchronize() if compute else synchronize())
        rb = _host.RouterHostReadback.decode(readback.ptr, top_k, tag)
    if rb is None:
        raise ShrikeError("router readback carries another launch's tag")  # RouterHostReadback.swift:47
    return rb


class BatchedDecodeLayer:
    """One MoE layer for a batch of tokens whose experts stream through a slot pool smaller than
    the expert set: the runner's loop around the operators (RealForwardRunner.swift:4552-4686 with
    the tile sequencing of PrefillRoutedTileSequencer). Router for all tokens, then passes: a
    pass plans as many of the still-unserved experts as the pool can take (shrike_amd.host.SlotCache),
    copies the misses from the pinned host store on the upload stream, and runs the grouped FFN
    for exactly that pass's experts; the token-major reduce and the shared expert close the layer.
    Everything numeric happens in libshrikehip; this class only sequences calls."""

    def __init__(self, moe: MoE, pool: ExpertPool, cache, offsets, host_store: PinnedBuffer, store_stride: int,
                 expert_bytes: int, max_tokens: int):
        d, f, ne, k = moe.desc.d, moe.desc.f, moe.desc.num_experts, moe.desc.top_k
        self.moe, self.pool, self.cache, self.off = moe, pool, cache, offsets
        self.store, self.store_stride, self.expert_bytes = host_store, store_stride, expert_bytes
        self.pf = Prefill(moe)
        self.upload_stream = Stream()
        self.t_max = max_tokens
        self.idx, self.w = empty(4 * max_tokens * k), empty(2 * max_tokens * k)
        self.router_ws = empty(self.pf.router_workspace_bytes(max_tokens, ne, d))
        self.routes = GroupedRoutesDevice(max_tokens * k, ne)
        self.partials = empty(2 * max_tokens * k * d)
        self.ffn_ws = empty(self.pf.ffn_workspace_bytes(max_tokens, self.routes.max_row_tiles))
        self.h2 = empty(2 * max_tokens * d)
        self.pass_table = empty(8 * ne)
        self.passes = 0
        self.plan_log = []  # every batch of experts handed to the cache, in order
        self.trace = None   # a list: run() then appends (stream name, start event, stop event) around what it enqueues

    def run(self, router, hidden, t: int, stride: int):
        """router: dict(weights, scales, biases, eff_scale, expert_scale, bias) of device buffers.
        Returns the device buffer h2[t, d]; self.idx / self.w hold the routes."""
        m, pf = self.moe, self.pf
        d, ne, k = m.desc.d, m.desc.num_experts, m.desc.top_k
        compute = m.stream

        def span(name, stream, body):
            if self.trace is None:
                return body()
            start, stop = Event(), Event()
            start.record(stream)
            out = body()
            stop.record(stream)
            self.trace.append((name, start, stop))
            return out
        span("compute", compute, lambda: pf.encode_block(
            router["weights"], router.get("scales"), router.get("biases"), hidden, router["eff_scale"],
            router["expert_scale"], router["bias"], self.idx, self.w, self.router_ws, t, ne, d, k, stride))
        (compute.synchronize() if compute else synchronize())
        ids = self.idx.download(np.uint32, t * k)  # the router's host readback
        # experts the pool already holds go first (PrefillSweepOrder.residentFirstBalanced), so a
        # step does not evict what it is about to use
        rows, last = {}, {}
        for i, e in enumerate(ids.tolist()):
            rows[e] = rows.get(e, 0) + 1
            last[e] = i // k
        resident = np.zeros(ne, np.uint8)
        resident[self.cache.resident_experts()] = 1
        todo = _host.resident_first_balanced(rows, last, resident, self.cache.slot_count, min(16, self.cache.slot_count))
        uploaded, served = Event(), Event()
        self.passes = 0
        while todo:
            batch = todo[: self.cache.slot_count]
            plan = self.cache.plan(batch)
            if plan is None:
                raise ShrikeError(capi.last_error())
            self.plan_log.append(list(batch))
            if self.passes:
                self.upload_stream.wait_event(served)  # the cells about to be overwritten were still being read
            span("upload", self.upload_stream, lambda: self.pool.execute_plan(
                self.cache, plan, self.store, self.store_stride, self.expert_bytes, self.upload_stream))
            # this pass's residency view: only its experts count as resident for the grouping
            table = np.full(ne, (capi.EMPTY << 32) | SENTINEL, np.uint64)
            for e in batch:
                table[e] = self.cache.entry(e)
            self.upload_stream.synchronize()  # the copy of `table` below reuses pageable memory
            self.pass_table.upload(table)
            uploaded.record(self.upload_stream)
            if compute:
                compute.wait_event(uploaded)
            def pass_kernels():
                pf.group_pairs(self.idx, self.w, t, k, ne, self.routes, residency=self.pass_table)
                pf.encode_grouped_expert_gemms(self.pool, self.off, self.routes, hidden, stride, self.partials, self.ffn_ws, t, k)
            span("compute", compute, pass_kernels)
            served.record(compute)
            (compute.synchronize() if compute else synchronize())
            todo = todo[len(batch):]
            self.passes += 1
        span("compute", compute, lambda: pf.encode_reduce_token_major(self.partials, self.w, self.h2, t, k, d))
        return self.h2


class StreamedPrefillLayer:
    """One prefill chunk's routed experts streamed from a layer file through a pool smaller than the
    chunk's expert set, sequenced the way the reference's ExpertStreamedTileDriver is
    (RealForwardRunner.swift:4698-4866 under PrefillRoutedTileSequencer.run): the chunk's expert groups
    are cut into tiles of `tile_experts`; a tile is planned against the slot cache (avoiding the cells
    that open and pending batches and a fetch in flight still hold, protecting the experts the chunk
    still needs), its misses are read by the parallel reader and copied to their cells on the upload
    stream, and once they have landed the grouped FFN runs for exactly that tile's experts on the compute
    stream. A batch of tiles is "committed" by recording an event and "drained" by waiting for it.
    Everything numeric happens in libshrikehip; this class only sequences calls."""

    def __init__(self, moe: MoE, pool: ExpertPool, cache, offsets, reader, file_offsets, blob_bytes: int,
                 staging: PinnedBuffer, max_tokens: int, config):
        d, ne, k = moe.desc.d, moe.desc.num_experts, moe.desc.top_k
        fitted = config.fitting(cache.slot_count)
        if fitted is None:
            raise ShrikeError(f"no tile configuration fits {cache.slot_count} slots")
        self.moe, self.pool, self.cache, self.off, self.config = moe, pool, cache, offsets, fitted
        self.reader, self.file_offsets, self.blob_bytes, self.staging = reader, list(file_offsets), blob_bytes, staging
        self.pf = Prefill(moe)
        self.upload_stream = Stream()
        self.idx, self.w = empty(4 * max_tokens * k), empty(2 * max_tokens * k)
        self.router_ws = empty(self.pf.router_workspace_bytes(max_tokens, ne, d))
        self.routes = GroupedRoutesDevice(max_tokens * k, ne)
        self.partials = empty(2 * max_tokens * k * d)
        self.ffn_ws = empty(self.pf.ffn_workspace_bytes(max_tokens, self.routes.max_row_tiles))
        self.h2 = empty(2 * max_tokens * d)
        self.trace = []  # (call, tile) in the order the sequencer made them

    def run(self, router, hidden, t: int, stride: int):
        m, pf = self.moe, self.pf
        d, ne, k = m.desc.d, m.desc.num_experts, m.desc.top_k
        compute = m.stream
        pf.encode_block(router["weights"], router.get("scales"), router.get("biases"), hidden, router["eff_scale"],
                        router["expert_scale"], router["bias"], self.idx, self.w, self.router_ws, t, ne, d, k, stride)
        (compute.synchronize() if compute else synchronize())
        ids, weights = self.idx.download(np.uint32, t * k), self.w.download(np.uint16, t * k)
        # experts the pool already holds go first (PrefillSweepOrder.residentFirstBalanced), so the chunk's first
        # tiles hit what the previous chunk left behind instead of evicting it
        rows, last = {}, {}
        for i, e in enumerate(ids.tolist()):
            rows[e] = rows.get(e, 0) + 1
            last[e] = i // k
        resident = np.zeros(ne, np.uint8)
        resident[self.cache.resident_experts()] = 1
        order = _host.resident_first_balanced(rows, last, resident, self.cache.slot_count, self.config.tile_experts)
        keys = _host.expert_sort_keys(order, ne)
        sort_keys = empty(8 * ne).upload(keys)
        grouped = _host.group_token_expert_pairs(_host.make_token_expert_pairs(ids, weights, t, k), t, k, ne,
                                                 tile_expert_count=self.config.tile_experts, expert_sort_keys=keys)
        self.grouped = grouped
        layer = self
        # one grouping for the chunk; every routed tile is then a pair range of it (encodeStreamedBatched)
        pf.group_pairs(self.idx, self.w, t, k, ne, self.routes, expert_sort_keys=sort_keys)

        class Driver:
            def __init__(self):
                self.protection = _host.ChunkExpertProtection([int(g["expert"]) for g in grouped.groups], ne)
                self.lifetime = _host.TileSlotLifetime()
                self.kept, self.begun = {}, {}
                self.open, self.pending = [], []  # open: (tile, slots, had misses, tile table); pending: (event, such entries)

            def experts_of(self, tile):
                tl = grouped.tiles[tile]
                return [int(g["expert"]) for g in grouped.groups[int(tl["group_start"]): int(tl["group_start"]) + int(tl["group_count"])]]

            open_batch_tiles = property(lambda self: len(self.open))
            open_batch_slots = property(lambda self: [s for entry in self.open for s in entry[1]])
            pending_depth = property(lambda self: len(self.pending))
            pending_assigned_slots = property(lambda self: [s for _, batch in self.pending for entry in batch for s in entry[1]])

            def _plan(self, tile, extra=()):
                experts = self.experts_of(tile)
                self.protection.planning(experts)
                avoiding = set(self.open_batch_slots) | set(self.pending_assigned_slots) | set(extra)
                return layer.cache.plan(experts, avoiding_slots=avoiding, protected_experts=self.protection.remaining)

            def plan(self, tile, avoiding_in_flight):
                layer.trace.append(("plan", tile))
                extra = ()
                if avoiding_in_flight is not None:
                    extra = self.begun[avoiding_in_flight][0].assigned_slots
                plan = self._plan(tile, extra)
                if plan is not None:
                    self.kept[tile] = plan
                return plan is not None

            def begin(self, tile):
                layer.trace.append(("begin", tile))
                plan = self.kept.pop(tile, None) or self._plan(tile)
                if plan is None:
                    raise ShrikeError(capi.last_error())
                slots, cells, experts = plan.assigned_slots, plan.assigned_cells, plan.experts
                miss_slots = [slots[i] for i in plan.misses]
                try:
                    if miss_slots:
                        layer.pool.fetch_experts(layer.reader, [layer.file_offsets[experts[i]] for i in plan.misses],
                                                 [cells[i] for i in plan.misses], layer.blob_bytes, layer.staging,
                                                 layer.upload_stream)
                except BaseException:
                    layer.cache.abandon(plan)
                    raise
                layer.cache.complete(plan)
                for expert, word in layer.cache.drain_publications():
                    layer.pool.publish(expert, word & 0xFFFFFFFF, word >> 32, layer.upload_stream)
                landed = Event()
                landed.record(layer.upload_stream)
                self.begun[tile] = (plan, landed)
                if miss_slots:
                    self.lifetime.begin(tile, miss_slots)

            def abandon_plan(self, tile):
                layer.trace.append(("abandonPlan", tile))
                plan = self.kept.pop(tile, None)
                if plan is not None:
                    layer.cache.abandon(plan)

            def encode(self, tile):
                layer.trace.append(("encode", tile))
                plan, landed = self.begun.pop(tile)
                table = np.full(ne, (capi.EMPTY << 32) | SENTINEL, np.uint64)
                for expert, cell in zip(plan.experts, plan.assigned_cells):
                    table[expert] = (capi.RESIDENT << 32) | cell
                landed.synchronize()  # the experts' bytes and words are in place; the table below is this tile's view
                tile_table = empty(8 * ne).upload(table)
                if compute:
                    compute.wait_event(landed)
                tl = grouped.tiles[tile]
                pf.encode_streamed_batched(layer.pool, layer.off, layer.routes, hidden, stride, layer.partials, layer.ffn_ws,
                                           t, k, int(tl["pair_start"]), int(tl["pair_count"]), residency=tile_table)
                self.open.append((tile, list(plan.assigned_slots), bool(plan.misses), tile_table))

            def commit_open_batch(self):
                if not self.open:
                    return
                layer.trace.append(("commit", None))
                done = Event()
                done.record(compute)
                self.pending.append((done, self.open))
                self.open = []

            def drain_oldest_batch(self):
                layer.trace.append(("drain", None))
                if not self.pending:
                    return
                done, batch = self.pending.pop(0)
                done.synchronize()
                for tile, _slots, missed, _table in batch:
                    if missed:
                        self.lifetime.complete(tile)

            def abandon_begun_fetches(self):
                layer.trace.append(("abandonBegun", None))
                layer.upload_stream.synchronize()
                self.begun.clear()
                for plan in self.kept.values():
                    layer.cache.abandon(plan)
                self.kept.clear()

        self.trace = []
        driver = Driver()
        _host.TileSequencer(_host.TileScheduler(self.config)).run(len(grouped.tiles), driver)
        pf.encode_reduce_token_major(self.partials, self.w, self.h2, t, k, d)
        return self.h2


class DecodeLayerWithMisses:
    """One token's routed experts when some of the selected experts are not in the pool: the runner's
    speculative pass and agreed fixup (RealForwardRunner.swift:2226-2294, :5115-5162, :5262-5283) over this
    build's operators. The classifier publishes four grids and a tagged readback; phase 1 runs for the hits
    and phase 2 only when nothing missed; the host reads the miss list, agrees a cell for every miss (the
    slot cache's plan for the selection: hits keep their cells, misses take victims outside it), writes the
    agreed row (the sentinel at the hits), has the missing blobs copied into their cells, and the fixup runs
    phase 1 over the agreed row and phase 2 over all positions, resolving a sentinel through that row.
    Everything numeric happens in libshrikehip; this class only sequences calls."""

    def __init__(self, moe: MoE, pool: ExpertPool, cache, offsets, host_store: PinnedBuffer, store_stride: int,
                 expert_bytes: int):
        k = moe.desc.top_k
        self.moe, self.pool, self.cache, self.off = moe, pool, cache, offsets
        self.store, self.store_stride, self.expert_bytes = host_store, store_stride, expert_bytes
        self.upload_stream = Stream()
        self.idx, self.w = empty(4 * 8), empty(2 * 8)
        self.resolved, self.agreed = empty(4 * 8), empty(4 * 8)
        self.hit_count, self.miss_count = empty(4), empty(4)
        self.hit_pos, self.miss_pos, self.miss_exp = empty(32), empty(32), empty(32)
        self.spec_args = empty(48)
        self.predicted = empty(4 * 8).fill(0)  # the runner's prediction for the next layer rides in the readback
        self.readback = PinnedBuffer(4 * (2 + 5 * k))
        self.acts = empty(2 * k * moe.desc.f)
        self.tag = 0
        self.fixups = 0

    def run(self, router, x, residual, y, hidden):
        """router: dict(weights, scales, biases, eff_scale, expert_scale, bias). x: fp16[d] (the router's and
        the experts' input), residual: fp16[d], y: fp16[d] out, hidden: fp16[d] updated in place."""
        m = self.moe
        d, f, ne, k = m.desc.d, m.desc.f, m.desc.num_experts, m.desc.top_k
        compute = m.stream
        m.encode_router(router["weights"], router.get("scales"), router.get("biases"), x, router["eff_scale"],
                        router["expert_scale"], router["bias"], self.idx, self.w, ne, d, k)
        self.tag = _host.RouterHostReadback.next_tag(self.tag)
        full = [1] * 12  # the operators below read only whether a grid's first word is zero
        m.encode_residency_classification(self.idx, self.pool.table, self.hit_count, self.hit_pos, self.miss_count,
                                          self.miss_pos, self.miss_exp, self.resolved, k, ne, full_grids=full,
                                          spec_args=self.spec_args, host_readback=self.readback, tag=self.tag,
                                          topk_weights=self.w, predicted=self.predicted)
        spec = self.spec_args.ptr
        m.encode_spec_phase1(self.pool, self.resolved, self.off, x, self.acts, d, f, k, indirect=spec)
        m.encode_spec_phase2(self.pool, self.resolved, self.off, self.acts, self.w, residual, y, hidden, d, f, k,
                             indirect=spec + 12)
        # the host reads the tagged words while the speculative launches still run
        rb = read_router_readback(self.readback, k, self.tag, compute)
        hits, misses = rb["hit_count"], rb["miss_count"]
        experts, miss_positions = rb["expert_ids"], rb["miss_positions"]
        if misses == 0:
            plan = self.cache.plan(experts)  # counts the hits, touches their recency
            self.cache.complete(plan)
            return
        plan = self.cache.plan(experts)
        if plan is None:
            raise ShrikeError(capi.last_error())
        if sorted(plan.misses) != sorted(miss_positions) or hits + misses != k:
            self.cache.abandon(plan)
            raise ShrikeError("the device's miss list and the slot cache disagree")
        row = np.full(8, SENTINEL, np.uint32)
        for i in plan.misses:
            row[i] = plan.assigned_cells[i]
        self.agreed.upload(row)
        self.pool.execute_plan(self.cache, plan, self.store, self.store_stride, self.expert_bytes, self.upload_stream)
        landed = Event()
        landed.record(self.upload_stream)
        if compute:
            compute.wait_event(landed)
        else:
            landed.synchronize()
        m.encode_spec_phase1(self.pool, self.agreed, self.off, x, self.acts, d, f, k, indirect=spec + 24)
        m.encode_spec_phase2(self.pool, self.resolved, self.off, self.acts, self.w, residual, y, hidden, d, f, k,
                             fallback_cells=self.agreed, indirect=spec + 36)
        self.fixups += 1


class AgreedDecodeLayer:
    """One token's routed experts over a pool of fewer slots than experts plus a prefetch ring: the runner's
    agreed layer (RealForwardRunner.swift:5262-5411) over this build's operators. Predictions are read ahead
    into ring cells as landings; the classifier sees a landed prediction as resident at its ring cell. After
    the speculative pass every miss of the classifier's list gets its cell: a landing the ring leased (no
    read), a free ring cell claimed as a landing, or, when the ring has none, a pool slot reserved as an
    overflow. The demand reads run on the storage threads; the fixup runs phase 1 over the agreed row and
    phase 2 over all positions; then the plan swaps every leased cell into the pool by index and the freed
    cells go back to the ring. All numerics happen in libshrikehip; this class sequences calls.

    `cache` is a shrike_amd.host.SlotCache made in a CellArena as long as the pool, `ring` an
    ExpertPrefetchRing over the cells behind the cache's slots (its drop callback must be this object's
    `drop_landing`), `layer` this layer's key in the ring. A begin for another layer reclaims this layer's
    finished landings that no route wanted, as in the runner."""

    JOIN_NANOS = 2_000_000

    def __init__(self, moe: MoE, pool: ExpertPool, cache, ring, offsets, host_store: PinnedBuffer, store_stride: int,
                 expert_bytes: int, scheduler, layer: int = 0):
        k = moe.desc.top_k
        self.moe, self.pool, self.cache, self.ring, self.off = moe, pool, cache, ring, offsets
        self.store, self.store_stride, self.expert_bytes = host_store, store_stride, expert_bytes
        self.scheduler, self.layer = scheduler, layer
        self.upload_stream = Stream()
        self.idx, self.w = empty(4 * 8), empty(2 * 8)
        self.resolved, self.agreed = empty(4 * 8), empty(4 * 8)
        self.hit_count, self.miss_count = empty(4), empty(4)
        self.hit_pos, self.miss_pos, self.miss_exp = empty(32), empty(32), empty(32)
        self.spec_args = empty(48)
        self.predicted = empty(4 * 8).fill(0)
        self.predicted_w = empty(2 * 8)
        self.predicted_next = []
        self.readback = PinnedBuffer(4 * (2 + 5 * k))
        self.acts = empty(2 * k * moe.desc.f)
        self.tag = 0
        self.fixups = self.overflows = self.landed_hits = self.demand_reads = 0
        # the demand batch's status word on the device and the three values it takes, in pinned memory
        self.status = empty(4).fill(0)
        self.status_values = PinnedBuffer(12)
        self.agreed_row = PinnedBuffer(32)
        self.status_values.array.view(np.uint32)[:] = (0, 1, 2)

    def drop_landing(self, layer: int, expert: int, cell: int) -> None:
        """The ring's reclaim of a landing no plan wanted (called with the ring locked)."""
        if layer == self.layer:
            self.cache.drop_landing(expert, cell)

    def _copy(self, experts, cells):
        """The reads: each expert's blob from the pinned store into its cell, enqueued on the upload stream. Returns
        the event recorded behind them; the bytes are in HBM once it has completed."""
        L = capi.load()
        for expert, cell in zip(experts, cells):
            check(L.shrike_hip_pool_upload_async(self.pool.handle, cell, self.store.ptr + expert * self.store_stride,
                                                 self.expert_bytes, self.upload_stream.handle),
                  "shrike_hip_pool_upload_async")
        landed = Event()
        landed.record(self.upload_stream)
        return landed

    def _store_status(self, value: int):
        """The batch's status word (ExpertIOCompletionToken.status: 0 loading, 1 complete, 2 failed), stored on the
        upload stream behind whatever was enqueued there."""
        check(capi.load().shrike_hip_memcpy_h2d_async(self.status.ptr, self.status_values.ptr + 4 * value, 4,
                                                      self.upload_stream.handle), "shrike_hip_memcpy_h2d_async")

    def _publish(self):
        """The cache's changed residency words into the device table, in order, ahead of the next launch."""
        for expert, word in self.cache.drain_publications():
            self.pool.publish(expert, word & 0xFFFFFFFF, word >> 32, self.moe.stream)

    def prefetch(self, predicted_experts) -> None:
        """schedulePredictivePrefetch (RealForwardRunner.swift:474-494) with beginPrefetch as the ring's issue
        (PreadExpertStreamer.swift:1034-1072): the predictions the pool lacks are claimed as landings in free
        ring cells and read speculatively; a refused or failed issue is counted, never thrown into the decode."""
        def issue(experts, cells):
            self.cache.claim_prefetch(experts, cells)  # PrefetchClaimRefused passes through to the ring
            operation = _host.ExpertLoadOperation()

            def work():
                operation.mark_in_flight()
                try:
                    self._copy(experts, cells).synchronize()
                    for expert, cell in zip(experts, cells):
                        self.cache.complete_landing(expert, cell)
                    operation.finish(0)
                except Exception:
                    for expert, cell in zip(experts, cells):
                        self.cache.fail_landing(expert, cell)
                    operation.finish(5)
            self.scheduler.submit(work, _host.ExpertIOScheduler.SPECULATIVE)
            return operation

        try:
            self.ring.begin(self.layer, list(predicted_experts), resident=self.cache.resident_experts(), issue=issue)
        except Exception:
            self.ring.note_hook_failure()

    def run(self, router, x, residual, y, hidden, probe=None):
        """router: dict(weights, scales, biases, eff_scale, expert_scale, bias). x: fp16[d], residual: fp16[d],
        y: fp16[d] out, hidden: fp16[d] updated in place. Returns the route's plan.
        probe: the following layer's router (same dict), or None. With it the router runs as the reference's pair
        (MoE.encodeRouterPair, RealForwardRunner.swift:2861): the second router over this layer's x names the experts
        the following layer is likely to want; they come back with the classifier's tagged readback and are left in
        `self.predicted_next` for the caller to hand to that layer's prefetch."""
        m = self.moe
        d, f, ne, k = m.desc.d, m.desc.f, m.desc.num_experts, m.desc.top_k
        compute = m.stream
        self._publish()
        if probe is None:
            m.encode_router(router["weights"], router.get("scales"), router.get("biases"), x, router["eff_scale"],
                            router["expert_scale"], router["bias"], self.idx, self.w, ne, d, k)
        else:
            def operands(r, out_indices, out_weights):
                return dict(weights=r["weights"], scales=r.get("scales"), biases=r.get("biases"),
                            effective_scale=r["eff_scale"], logit_bias=r["bias"], out_indices=out_indices, out_weights=out_weights)
            m.encode_router_pair(operands(router, self.idx, self.w), operands(probe, self.predicted, self.predicted_w), x,
                                 router["expert_scale"], ne, d, k)
        self.tag = _host.RouterHostReadback.next_tag(self.tag)
        m.encode_residency_classification(self.idx, self.pool.table, self.hit_count, self.hit_pos, self.miss_count,
                                          self.miss_pos, self.miss_exp, self.resolved, k, ne, full_grids=[1] * 12,
                                          spec_args=self.spec_args, host_readback=self.readback, tag=self.tag,
                                          topk_weights=self.w, predicted=self.predicted)
        spec = self.spec_args.ptr
        m.encode_spec_phase1(self.pool, self.resolved, self.off, x, self.acts, d, f, k, indirect=spec)
        m.encode_spec_phase2(self.pool, self.resolved, self.off, self.acts, self.w, residual, y, hidden, d, f, k,
                             indirect=spec + 12)
        rb = read_router_readback(self.readback, k, self.tag, compute)  # polled while the speculative launches run
        misses, experts, miss_positions = rb["miss_count"], rb["expert_ids"], rb["miss_positions"]
        self.predicted_next = rb["predicted_ids"] if probe is not None else []

        # joinAgreedLandings, :5262-5267
        leased = self.ring.ready_cells(self.layer, experts, self.JOIN_NANOS)
        # agreeCells / agreeCell, :5273-5317
        unleased = [experts[p] for p in miss_positions if experts[p] not in leased]
        claimed = self.ring.claim_demand(self.layer, unleased)
        read_experts, read_cells, overflow = [], [], {}
        row = np.full(8, SENTINEL, np.uint32)
        try:
            for position in miss_positions:
                expert = experts[position]
                if expert in leased:
                    row[position] = leased[expert]
                    continue
                if expert in claimed:
                    if self.cache.claim_landing(expert, claimed[expert]):
                        read_experts.append(expert)
                        read_cells.append(claimed[expert])
                        row[position] = claimed[expert]
                        continue
                    self.ring.consume(self.layer, [expert], {})
                    del claimed[expert]
                late = self.ring.ready_cells(self.layer, [expert], self.JOIN_NANOS)
                if expert in late:
                    leased[expert] = row[position] = late[expert]
                    continue
                cell = self.cache.reserve_overflow_slot(expert, protecting=experts)
                if cell is None:
                    raise ShrikeError(f"layer {self.layer} has no cell for expert {expert}")  # expertCacheUnplaceable
                overflow[expert] = cell
                read_experts.append(expert)
                read_cells.append(cell)
                row[position] = cell
        except Exception:
            # abandonAgreedContext, :5342-5349
            self.ring.consume(self.layer, list(set(leased) | set(claimed)), {})
            for expert, cell in overflow.items():
                self.cache.abandon_overflow_slot(expert, cell)
            raise
        self.overflows += len(overflow)

        # submitAgreedReads, :5319-5340 (beginAgreedReads, PreadExpertStreamer.swift:903-964)
        # The storage thread enqueues the copies, the status word and an event on the upload stream and finishes the
        # operation once they are enqueued; the compute stream then waits for that event ahead of the fixup
        # launches, which read the status word (moe.metal:36-39). What the host waits for is the enqueue, not the
        # bytes: the wait for them is the GPU's, as with the reference's encodeWaitForEvent
        # (RealForwardRunner.swift:5124, ExpertIOEventCoordinator.swift:76-89).
        operation = _host.ExpertLoadOperation()
        uploaded = []
        if read_experts:
            started = _host.monotonic_nanos()
            self._store_status(0)

            def work():
                operation.mark_in_flight()
                fetch_started = _host.monotonic_nanos()
                try:
                    copies = self._copy(read_experts, read_cells)
                    self._store_status(1)
                    landed = Event()
                    landed.record(self.upload_stream)
                    uploaded.append(landed)
                    del copies
                    enqueued = _host.monotonic_nanos()
                    self.cache.finish_agreed_reads(read_experts, read_cells, True, enqueued - started, enqueued - fetch_started)
                    operation.finish(0)
                except Exception:
                    try:
                        self._store_status(2)
                    except Exception:
                        pass
                    self.cache.finish_agreed_reads(read_experts, read_cells, False)
                    operation.finish(5)
            self.scheduler.submit(work, _host.ExpertIOScheduler.DEMAND)
            self.ring.attach_demand(self.layer, list(claimed), operation)
            self.ring.note_demand_submission()
            self.demand_reads += len(read_experts)
        else:
            operation.finish(0)

        held = list(set(leased) | set(claimed))
        if misses:
            try:
                operation.wait()  # until the batch is enqueued on the upload stream (or has failed)
            except Exception:
                self.ring.consume(self.layer, held, {})  # abandonPendingAgreedLayer, :5351-5355
                raise ShrikeError(f"layer {self.layer}: an agreed read failed")
            if compute:  # the agreed row goes out on the compute stream: a blocking copy would wait for the upload stream too
                self.agreed_row.array.view(np.uint32)[:] = row
                check(capi.load().shrike_hip_memcpy_h2d_async(self.agreed.ptr, self.agreed_row.ptr, 32, compute.handle),
                      "shrike_hip_memcpy_h2d_async")
            else:
                self.agreed.upload(row)
            self._publish()
            io_status = None
            if uploaded:
                if compute:
                    compute.wait_event(uploaded[0])  # the GPU waits for the bytes; the host goes on encoding
                else:
                    uploaded[0].synchronize()        # the null stream has no handle to wait on
                io_status = self.status
            m.encode_spec_phase1(self.pool, self.agreed, self.off, x, self.acts, d, f, k, indirect=spec + 24,
                                 io_status=io_status)
            m.encode_spec_phase2(self.pool, self.resolved, self.off, self.acts, self.w, residual, y, hidden, d, f, k,
                                 fallback_cells=self.agreed, indirect=spec + 36, io_status=io_status)
            self.fixups += 1

        # planAgreedLayer, :5380-5411
        miss_experts = [experts[p] for p in miss_positions]
        plan = self.cache.plan(experts, gpu_missed_experts=miss_experts, leased_landings=held,
                               misses_counted=len(read_experts))
        if plan is None:
            self.ring.unlease(self.layer, held)
            raise ShrikeError(f"layer {self.layer}: the route does not fit its pool")
        if plan.misses:
            self.cache.abandon(plan)
            self.ring.consume(self.layer, held, plan.freed_cells)
            raise ShrikeError(f"layer {self.layer}: an agreed read did not land for experts "
                              f"{[plan.experts[i] for i in plan.misses]}")
        self.landed_hits += sum(1 for e in leased if e not in miss_experts)
        self.ring.consume(self.layer, held, plan.freed_cells)
        self._publish()
        return plan
