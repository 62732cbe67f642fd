"""Thin Python face of the C ABI for tests, the smoke run and the benchmark.

Everything runs through libshrikehip (include/shrike_hip.h): device memory, streams
and events come from its plumbing calls, host arrays are numpy. No other GPU
runtime is loaded, and nothing here computes on the CPU.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import capi
from . import host as _host
from .capi import (ACT_SILU, META_BF16, SENTINEL, DecodeLayerArgs, ExpertOffsets, MoEDesc,
                   PoolBases, Projection, ShrikeError, check)

_initialised = False


def gpu_available() -> bool:
    """True when device 0 is a gfx950 GPU this process can use."""
    try:
        return capi.load().shrike_hip_init(0) == 0
    except (OSError, ShrikeError):
        return False


def init(device: int = 0) -> None:
    global _initialised
    if not _initialised:
        check(capi.load().shrike_hip_init(device), "shrike_hip_init")
        _initialised = True


def synchronize() -> None:
    check(capi.load().shrike_hip_device_synchronize(), "shrike_hip_device_synchronize")


class DeviceBuffer:
    """A device allocation; `.ptr` is the device address."""

    def __init__(self, nbytes: int):
        init()
        self.nbytes = int(nbytes)
        self.ptr = capi.load().shrike_hip_malloc(self.nbytes)
        if not self.ptr:
            raise ShrikeError(capi.last_error())

    def upload(self, a: np.ndarray, offset: int = 0) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        assert offset + a.nbytes <= self.nbytes
        check(capi.load().shrike_hip_memcpy_h2d(self.ptr + offset, a.ctypes.data, a.nbytes), "memcpy_h2d")
        return self

    def download(self, dtype, count: int | None = None, offset: int = 0) -> np.ndarray:
        dtype = np.dtype(dtype)
        n = (self.nbytes - offset) // dtype.itemsize if count is None else count
        out = np.empty(n, dtype)
        check(capi.load().shrike_hip_memcpy_d2h(out.ctypes.data, self.ptr + offset, out.nbytes), "memcpy_d2h")
        return out

    def fill(self, byte: int = 0) -> "DeviceBuffer":
        check(capi.load().shrike_hip_memset(self.ptr, byte, self.nbytes), "memset")
        return self

    def free(self) -> None:
        if self.ptr:
            capi.load().shrike_hip_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def dev(a: np.ndarray) -> DeviceBuffer:
    a = np.ascontiguousarray(a)
    return DeviceBuffer(max(a.nbytes, 16)).upload(a)


def empty(nbytes: int) -> DeviceBuffer:
    return DeviceBuffer(max(nbytes, 16)).fill(0)


def ptr(b) -> int | None:
    if b is None:
        return None
    return b.ptr if isinstance(b, (DeviceBuffer, PinnedBuffer)) else int(b)


class PinnedBuffer:
    """Page-locked host memory from the library (hipHostMalloc), viewed as a numpy array."""

    def __init__(self, nbytes: int):
        init()
        self.nbytes = int(nbytes)
        self.ptr = capi.load().shrike_hip_host_alloc(self.nbytes)
        if not self.ptr:
            raise ShrikeError(f"shrike_hip_host_alloc({nbytes}) failed: {capi.last_error()}")
        self.array = np.ctypeslib.as_array((C.c_uint8 * self.nbytes).from_address(self.ptr))

    def free(self):
        if self.ptr:
            self.array = None
            capi.load().shrike_hip_host_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Stream:
    def __init__(self):
        init()
        self.handle = capi.load().shrike_hip_stream_create()
        if not self.handle:
            raise ShrikeError(capi.last_error())

    def synchronize(self):
        check(capi.load().shrike_hip_stream_synchronize(self.handle), "stream_synchronize")

    def wait_event(self, event: "Event"):
        check(capi.load().shrike_hip_stream_wait_event(self.handle, event.handle), "stream_wait_event")

    def close(self):
        if self.handle:
            capi.load().shrike_hip_stream_destroy(self.handle)
            self.handle = None


class Event:
    def __init__(self):
        init()
        self.handle = capi.load().shrike_hip_event_create()
        if not self.handle:
            raise ShrikeError(capi.last_error())

    def record(self, stream: Stream | None = None):
        check(capi.load().shrike_hip_event_record(self.handle, stream.handle if stream else None), "event_record")

    def synchronize(self):
        check(capi.load().shrike_hip_event_synchronize(self.handle), "event_synchronize")

    def elapsed_ms(self, later: "Event") -> float:
        ms = C.c_float(0)
        check(capi.load().shrike_hip_event_elapsed_ms(self.handle, later.handle, C.byref(ms)), "event_elapsed")
        return ms.value

    def close(self):
        """Destroys the event (work already enqueued that waits for it is not affected)."""
        if self.handle:
            capi.load().shrike_hip_event_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def expert_offsets(d: int, f: int, bits: int = 4, additive_biases: bool = False):
    off = ExpertOffsets()
    stride = capi.load().shrike_expert_offsets_make(d, f, bits, int(additive_biases), C.byref(off))
    if stride == 0:
        raise ShrikeError(capi.last_error())
    return off, stride


class ExpertPool:
    """shrike_hip_pool: the HBM cell arena and residency table of one layer."""

    def __init__(self, cells: int, expert_stride: int, num_experts: int, chunk_bytes: int = 0):
        init()
        err = C.c_int(0)
        L = capi.load()
        self.handle = L.shrike_hip_pool_create(cells, expert_stride, num_experts, chunk_bytes, C.byref(err))
        if not self.handle:
            raise ShrikeError(f"shrike_hip_pool_create failed with {err.value}: {capi.last_error()}")
        self.cells, self.num_experts = cells, num_experts
        self.stride = L.shrike_hip_pool_slot_stride(self.handle)
        self.bases = L.shrike_hip_pool_bases(self.handle)
        self.table = L.shrike_hip_pool_residency_table(self.handle)

    def layer_view(self, num_experts: int | None = None) -> "ExpertPool":
        """Another layer's residency table over this pool's cells (one arena for the model, a table per layer);
        this pool must outlive the view."""
        err = C.c_int(0)
        L = capi.load()
        view = object.__new__(ExpertPool)
        view.handle = L.shrike_hip_pool_create_layer_view(self.handle, num_experts or self.num_experts, C.byref(err))
        if not view.handle:
            raise ShrikeError(f"shrike_hip_pool_create_layer_view failed with {err.value}: {capi.last_error()}")
        view.cells, view.num_experts = self.cells, num_experts or self.num_experts
        view.stride, view.bases = self.stride, L.shrike_hip_pool_bases(view.handle)
        view.table = L.shrike_hip_pool_residency_table(view.handle)
        view._arena = self  # keeps the cells alive
        return view

    def cell_ptr(self, cell: int) -> int:
        p = capi.load().shrike_hip_pool_cell_ptr(self.handle, cell)
        if not p:
            raise ShrikeError(capi.last_error())
        return p

    def upload(self, cell: int, blob: np.ndarray, stream: Stream | None = None) -> None:
        blob = np.ascontiguousarray(blob)
        check(capi.load().shrike_hip_pool_upload_async(self.handle, cell, blob.ctypes.data, blob.nbytes,
                                                       stream.handle if stream else None),
              "shrike_hip_pool_upload_async")
        synchronize()  # the source is pageable host memory owned by numpy

    def publish(self, expert: int, cell: int, state: int, stream: Stream | None = None) -> None:
        check(capi.load().shrike_hip_pool_table_publish(self.handle, expert, cell, state,
                                                        stream.handle if stream else None),
              "shrike_hip_pool_table_publish")

    def entry(self, expert: int) -> int:
        return capi.load().shrike_hip_pool_table_entry(self.handle, expert)

    def execute_plan(self, cache, plan, host_store, store_expert_stride: int, expert_bytes: int,
                     stream: Stream | None = None, elapsed_nanos: int = 0) -> None:
        """executeExpertCachePlan: copy the plan's misses from the pinned host store into their cells,
        mark them resident and store the changed residency words, all on `stream`. `cache` is a
        shrike_amd.host.SlotCache, `plan` its CachePlan."""
        check(capi.load().shrike_hip_pool_execute_plan(self.handle, cache._h, C.byref(plan.c), ptr(host_store),
                                                       store_expert_stride, expert_bytes,
                                                       stream.handle if stream else None, elapsed_nanos),
              "shrike_hip_pool_execute_plan")

    def fetch_experts(self, reader, file_offsets, cells, blob_bytes: int, staging: "PinnedBuffer",
                      stream: Stream | None = None) -> None:
        """Blobs at file_offsets of the reader's layer file -> cells, through the pinned staging buffer.
        `reader` is a shrike_amd.host.ParallelExpertReader created with stride blob_bytes."""
        n = len(file_offsets)
        offs = (C.c_uint64 * n)(*[int(o) for o in file_offsets])
        cs = (C.c_uint32 * n)(*[int(c) for c in cells])
        check(capi.load().shrike_hip_pool_fetch_experts(self.handle, stream.handle if stream else None, reader.handle,
                                                        offs, cs, n, blob_bytes, staging.ptr, staging.nbytes),
              "shrike_hip_pool_fetch_experts")

    def close(self) -> None:
        if self.handle:
            capi.load().shrike_hip_pool_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class MoE:
    """shrike_hip_moe with the reference's operator names (sources/Shrike/Kernels/MoE/MoE.swift)."""

    def __init__(self, d, f, num_experts, top_k, routed_bits=4, router_bits=0, meta=META_BF16,
                 activation=ACT_SILU, additive_biases=False, sigmoid=False, scaling=1.0,
                 event_gated=False):
        init()
        self.desc = MoEDesc(d, f, num_experts, top_k, routed_bits, router_bits, meta, activation,
                            int(additive_biases), int(sigmoid), float(scaling), int(event_gated))
        err = C.c_int(0)
        self.handle = capi.load().shrike_hip_moe_create(C.byref(self.desc), C.byref(err))
        if not self.handle:
            raise ShrikeError(f"shrike_hip_moe_create failed with {err.value}: {capi.last_error()}")
        self.stream: Stream | None = None  # None = the default stream

    def _s(self):
        return self.stream.handle if self.stream else None

    def close(self):
        if self.handle:
            capi.load().shrike_hip_moe_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def logits(self, num_experts: int) -> np.ndarray:
        synchronize()
        out = np.empty(num_experts, np.float32)
        p = capi.load().shrike_hip_moe_router_logits(self.handle)
        check(capi.load().shrike_hip_memcpy_d2h(out.ctypes.data, p, out.nbytes), "memcpy_d2h")
        return out

    def encode_router(self, weights, scales, biases, hidden, effective_scale, per_expert_scale,
                      logit_bias, out_indices, out_weights, num_experts, d, top_k):
        check(capi.load().shrike_hip_moe_router(
            self.handle, self._s(), ptr(weights), ptr(scales), ptr(biases), ptr(hidden),
            ptr(effective_scale), ptr(per_expert_scale), ptr(logit_bias), ptr(out_indices),
            ptr(out_weights), num_experts, d, top_k), "shrike_hip_moe_router")

    def encode_router_pair(self, first: dict, second: dict, hidden, per_expert_scale, num_experts, d, top_k,
                           second_logits=None):
        """MoE.encodeRouterPair: first/second are dicts with weights, scales, biases, effective_scale, logit_bias,
        out_indices, out_weights (device buffers; scales/biases None for fp16 rows)."""
        def ops(o):
            return capi.RouterOperands(*(ptr(o.get(n)) for n in ("weights", "scales", "biases", "effective_scale",
                                                                   "logit_bias", "out_indices", "out_weights")))
        a, b = ops(first), ops(second)
        check(capi.load().shrike_hip_moe_router_pair(
            self.handle, self._s(), C.byref(a), C.byref(b), ptr(hidden), ptr(per_expert_scale), num_experts, d, top_k,
            ptr(second_logits)), "shrike_hip_moe_router_pair")

    def pair_logits(self, num_experts: int) -> np.ndarray:
        synchronize()
        out = np.empty(num_experts, np.float32)
        p = capi.load().shrike_hip_moe_router_pair_logits(self.handle)
        check(capi.load().shrike_hip_memcpy_d2h(out.ctypes.data, p, out.nbytes), "memcpy_d2h")
        return out

    def encode_residency_classification(self, topk, residency, hit_count, hit_positions, miss_count,
                                        miss_positions, miss_experts, resolved_slots, top_k, num_experts,
                                        full_grids=None, spec_args=None, host_readback=None, tag=0,
                                        topk_weights=None, predicted=None):
        grids = (C.c_uint32 * 12)(*(full_grids if full_grids is not None else [1] * 12))
        check(capi.load().shrike_hip_moe_classify(
            self.handle, self._s(), ptr(topk), ptr(residency), ptr(hit_count), ptr(hit_positions),
            ptr(miss_count), ptr(miss_positions), ptr(miss_experts), ptr(resolved_slots), top_k,
            num_experts, grids, ptr(spec_args), ptr(host_readback), tag, ptr(topk_weights),
            ptr(predicted)), "shrike_hip_moe_classify")

    def encode_spec_phase1(self, pool: ExpertPool, resolved_slots, offsets, x, acts, d, f, top_k,
                           indirect=None, io_status=None):
        check(capi.load().shrike_hip_moe_phase1_pool(
            self.handle, self._s(), pool.bases, pool.stride, ptr(resolved_slots), C.byref(offsets),
            ptr(x), ptr(acts), d, f, top_k, ptr(indirect), ptr(io_status)), "shrike_hip_moe_phase1_pool")

    def encode_spec_phase2(self, pool: ExpertPool, resolved_slots, offsets, acts, routing_weights,
                           residual, y, hidden, d, f, top_k, fallback_cells=None, indirect=None,
                           io_status=None):
        check(capi.load().shrike_hip_moe_phase2_pool(
            self.handle, self._s(), pool.bases, pool.stride, ptr(resolved_slots), ptr(fallback_cells),
            C.byref(offsets), ptr(acts), ptr(routing_weights), ptr(residual), ptr(y), ptr(hidden),
            d, f, top_k, ptr(indirect), ptr(io_status)), "shrike_hip_moe_phase2_pool")

    def make_routed_argument_buffer(self, blob_ptrs, buffer: "DeviceBuffer | None" = None) -> "DeviceBuffer":
        """MoE.makeReusedRoutedArgumentBuffer (MoE.swift:612-620): the device array of the route's blob pointers."""
        words = np.asarray(list(blob_ptrs), np.uint64)
        buffer = buffer or empty(8 * capi.MAX_TOP_K).fill(0)
        buffer.upload(words)
        return buffer

    def encode_routed_persistent_phase1(self, routed_arg_buffer, offsets, x, acts, d, f, top_k, active_slots=None,
                                        active_count=0, io_status=None):
        """encodeRoutedPersistentPhase1U16Load, and with active_slots encodeRoutedPersistentPhase1SubsetU16Load."""
        check(capi.load().shrike_hip_moe_phase1_blobs(
            self.handle, self._s(), ptr(routed_arg_buffer), C.byref(offsets), ptr(x), ptr(acts), d, f, top_k,
            ptr(active_slots), active_count, ptr(io_status)), "shrike_hip_moe_phase1_blobs")

    def encode_routed_persistent_phase2(self, routed_arg_buffer, offsets, acts, routing_weights, residual, y, hidden,
                                        d, f, top_k, io_status=None):
        """encodeRoutedPersistentPhase2Reduce."""
        check(capi.load().shrike_hip_moe_phase2_blobs(
            self.handle, self._s(), ptr(routed_arg_buffer), C.byref(offsets), ptr(acts), ptr(routing_weights),
            ptr(residual), ptr(y), ptr(hidden), d, f, top_k, ptr(io_status)), "shrike_hip_moe_phase2_blobs")

    def encode_resolve_batch(self, topk, residency, resolved_slots, count, num_experts, miss_count=None):
        check(capi.load().shrike_hip_moe_resolve_batch(self._s(), ptr(topk), ptr(residency), ptr(resolved_slots), count,
                                                       num_experts, ptr(miss_count)), "shrike_hip_moe_resolve_batch")

    def encode_phase1_batch(self, pool: ExpertPool, resolved_slots, offsets, x, x_stride, acts, d, f, top_k, tokens):
        check(capi.load().shrike_hip_moe_phase1_batch(self.handle, self._s(), pool.bases, pool.stride, ptr(resolved_slots),
                                                      C.byref(offsets), ptr(x), x_stride, ptr(acts), d, f, top_k, tokens),
              "shrike_hip_moe_phase1_batch")

    def encode_phase2_batch(self, pool: ExpertPool, resolved_slots, offsets, acts, routing_weights, residual, y, hidden,
                            d, f, top_k, tokens):
        check(capi.load().shrike_hip_moe_phase2_batch(self.handle, self._s(), pool.bases, pool.stride, ptr(resolved_slots),
                                                      C.byref(offsets), ptr(acts), ptr(routing_weights), ptr(residual), ptr(y),
                                                      ptr(hidden), d, f, top_k, tokens), "shrike_hip_moe_phase2_batch")

    def encode_shared_expert(self, gate, up, down, bits, x, scratch, h1, d, f_shared, scalar_gate=None):
        def proj(t):
            return Projection(ptr(t[0]), ptr(t[1]), ptr(t[2]))
        g, u, dn = proj(gate), proj(up), proj(down)
        check(capi.load().shrike_hip_shared_expert(
            self.handle, self._s(), C.byref(g), C.byref(u), C.byref(dn), bits, ptr(x), ptr(scratch),
            ptr(h1), ptr(scalar_gate), d, f_shared), "shrike_hip_shared_expert")

    def encode_decode_layer(self, args: DecodeLayerArgs):
        check(capi.load().shrike_hip_moe_decode_layer(self.handle, self._s(), C.byref(args)),
              "shrike_hip_moe_decode_layer")

    def encode_decode_layer_launches(self, args: DecodeLayerArgs, launches: int):
        """A subset of the layer's three launches (bit 0 head, bit 1 phase 1, bit 2 phase 2)."""
        check(capi.load().shrike_hip_moe_decode_layer_launches(self.handle, self._s(), C.byref(args), launches),
              "shrike_hip_moe_decode_layer_launches")


class GroupedRoutesDevice:
    """Device buffers of shrike_hip_grouped_routes for up to `pairs` pairs over `num_experts`."""

    def __init__(self, pairs: int, num_experts: int):
        self.pairs, self.num_experts = pairs, num_experts
        self.max_row_tiles = capi.load().shrike_hip_group_max_row_tiles(pairs, num_experts)
        self.sorted_pairs = empty(max(1, pairs) * 16)
        self.offsets = empty(num_experts * 4)
        self.counts = empty(num_experts * 4)
        self.row_tiles = empty(max(1, self.max_row_tiles) * 16)
        self.row_tile_count = empty(4).fill(0)
        self.c = capi.HipGroupedRoutes(ptr(self.sorted_pairs), ptr(self.offsets), ptr(self.counts),
                                       ptr(self.row_tiles), ptr(self.row_tile_count))

    def download(self):
        n = int(self.row_tile_count.download(np.uint32, 1)[0])
        return dict(sorted_pairs=self.sorted_pairs.download(np.uint32, self.pairs * 4).reshape(-1, 4),
                    offsets=self.offsets.download(np.uint32, self.num_experts),
                    counts=self.counts.download(np.uint32, self.num_experts),
                    row_tiles=self.row_tiles.download(np.uint32, n * 4).reshape(-1, 4), row_tile_count=n)


class Prefill:
    """The prefill operators of the routed path with the reference's names: PrefillRouter.encodeBlock,
    PrefillMoEGrouping on the device, PrefillGroupedRoutedMoE.encodeGroupedExpertGEMMs,
    PrefillMoE.encodeReduceTokenMajor."""

    def __init__(self, moe: MoE):
        self.moe = moe

    def _s(self):
        return self.moe._s()

    def router_workspace_bytes(self, query_count, num_experts, d):
        return capi.load().shrike_hip_prefill_router_workspace_bytes(query_count, num_experts, d)

    def encode_block(self, weights, scales, biases, hidden, effective_scale, per_expert_scale, logit_bias,
                     out_indices, out_weights, logits_workspace, query_count, num_experts, d, top_k,
                     hidden_stride_elements):
        check(capi.load().shrike_hip_prefill_router(
            self.moe.handle, self._s(), ptr(weights), ptr(scales), ptr(biases), ptr(hidden), ptr(effective_scale),
            ptr(per_expert_scale), ptr(logit_bias), ptr(out_indices), ptr(out_weights), ptr(logits_workspace),
            query_count, num_experts, d, top_k, hidden_stride_elements), "shrike_hip_prefill_router")

    def group_pairs(self, indices, weights, query_count, top_k, num_experts, routes: GroupedRoutesDevice,
                    expert_sort_keys=None, residency=None):
        check(capi.load().shrike_hip_group_pairs(self._s(), ptr(indices), ptr(weights), query_count, top_k, num_experts,
                                                 ptr(expert_sort_keys), ptr(residency), C.byref(routes.c)),
              "shrike_hip_group_pairs")

    def ffn_workspace_bytes(self, query_count, max_row_tiles):
        return capi.load().shrike_hip_prefill_ffn_workspace_bytes(query_count, max_row_tiles, self.moe.desc.d,
                                                                  self.moe.desc.f)

    def encode_grouped_expert_gemms(self, pool: ExpertPool, offsets, routes: GroupedRoutesDevice, hidden,
                                    hidden_stride_elements, route_partials, workspace: DeviceBuffer, query_count,
                                    top_k, max_row_tiles=None):
        check(capi.load().shrike_hip_prefill_grouped_ffn(
            self.moe.handle, self._s(), pool.bases, pool.stride, C.byref(offsets), C.byref(routes.c),
            routes.max_row_tiles if max_row_tiles is None else max_row_tiles, ptr(hidden), hidden_stride_elements,
            ptr(route_partials), ptr(workspace), workspace.nbytes, query_count, self.moe.desc.d, self.moe.desc.f, top_k),
            "shrike_hip_prefill_grouped_ffn")

    def encode_streamed_batched(self, pool: ExpertPool, offsets, routes: GroupedRoutesDevice, hidden,
                                hidden_stride_elements, route_partials, workspace: DeviceBuffer, query_count, top_k,
                                pair_start: int, pair_count: int, residency=None, pair_microbatch_rows: int = 32,
                                max_row_tiles=None) -> int:
        """encodeStreamedBatched (PrefillGroupedRoutedMoE.swift:846-922): the routed FFN of the sorted pairs
        [pair_start, pair_start + pair_count) against `residency` (a device table, default the cells recorded at
        grouping); returns the reference's microbatch count."""
        count = C.c_uint32(0)
        check(capi.load().shrike_hip_prefill_streamed_batched(
            self.moe.handle, self._s(), pool.bases, pool.stride, C.byref(offsets), C.byref(routes.c),
            routes.max_row_tiles if max_row_tiles is None else max_row_tiles, ptr(residency), pair_start, pair_count,
            pair_microbatch_rows, ptr(hidden), hidden_stride_elements, ptr(route_partials), ptr(workspace),
            workspace.nbytes, query_count, self.moe.desc.d, self.moe.desc.f, top_k, C.byref(count)),
            "shrike_hip_prefill_streamed_batched")
        return count.value

    def encode_shared_expert(self, gate, up, down, bits, hidden, hidden_stride_elements, h1, query_count, f_shared,
                             workspace: DeviceBuffer | None = None, scalar_gate=None):
        """The shared expert for every token of the chunk; returns the workspace it used."""
        need = capi.load().shrike_hip_prefill_shared_expert_workspace_bytes(query_count, self.moe.desc.d, f_shared)
        if workspace is None or workspace.nbytes < need:
            workspace = empty(need)
        g, u, dn = (Projection(ptr(t[0]), ptr(t[1]), ptr(t[2])) for t in (gate, up, down))
        check(capi.load().shrike_hip_prefill_shared_expert(
            self.moe.handle, self._s(), C.byref(g), C.byref(u), C.byref(dn), bits, ptr(hidden), hidden_stride_elements,
            ptr(h1), ptr(scalar_gate), ptr(workspace), workspace.nbytes, query_count, self.moe.desc.d, f_shared),
            "shrike_hip_prefill_shared_expert")
        return workspace

    def encode_scalar_gate_rows(self, gate_row, x, x_stride_elements, gate, rows, d):
        """Elementwise.encodeScalarGateRows: gate_row is the (weights, scales, biases) of the one 8-bit row."""
        g = Projection(ptr(gate_row[0]), ptr(gate_row[1]), ptr(gate_row[2]))
        check(capi.load().shrike_hip_shared_scalar_gate_rows(self._s(), C.byref(g), self.moe.desc.meta_dtype, ptr(x),
                                                             x_stride_elements, ptr(gate), rows, d),
              "shrike_hip_shared_scalar_gate_rows")

    def encode_sigmoid_scalar_mul_rows(self, y, gate, d, rows):
        check(capi.load().shrike_hip_sigmoid_scalar_mul_rows(self._s(), ptr(y), ptr(gate), d, rows),
              "shrike_hip_sigmoid_scalar_mul_rows")

    def encode_reduce_token_major(self, route_partials, route_weights, h2, query_count, top_k, d):
        check(capi.load().shrike_hip_prefill_reduce(self._s(), ptr(route_partials), ptr(route_weights), ptr(h2),
                                                    query_count, top_k, d), "shrike_hip_prefill_reduce")

    def residual_add(self, hidden, delta, count):
        check(capi.load().shrike_hip_residual_add_f16(self._s(), ptr(hidden), ptr(delta), count),
              "shrike_hip_residual_add_f16")


def residual_add_rmsnorm_bf16w(hidden, delta, weight, out, d: int, eps: float, rows: int = 1,
                               stream: Stream | None = None) -> None:
    """RMSNorm.encodeResidualAddBF16W (delta None: encodeBF16W): hidden += delta in place, out = the
    normalised row the router, the shared expert and phase 1 read."""
    check(capi.load().shrike_hip_residual_add_rmsnorm_bf16w(stream.handle if stream else None, ptr(hidden), ptr(delta),
                                                            ptr(weight), ptr(out), d, eps, rows),
          "shrike_hip_residual_add_rmsnorm_bf16w")


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

    def run(self, router, hidden, t: int, stride: int):
        """router: dict(weights, scales, biases, eff_scale, expert_scale, bias) of device buffers.
        Returns the device buffer h2[t, d]; self.idx / self.w hold the routes."""
        m, pf = self.moe, self.pf
        d, ne, k = m.desc.d, m.desc.num_experts, m.desc.top_k
        compute = m.stream
        pf.encode_block(router["weights"], router.get("scales"), router.get("biases"), hidden, router["eff_scale"],
                        router["expert_scale"], router["bias"], self.idx, self.w, self.router_ws, t, ne, d, k, stride)
        (compute.synchronize() if compute else synchronize())
        ids = self.idx.download(np.uint32, t * k)  # the router's host readback
        # experts the pool already holds go first (PrefillSweepOrder.residentFirstBalanced), so a
        # step does not evict what it is about to use
        from . import host as _host
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
            self.pool.execute_plan(self.cache, plan, self.store, self.store_stride, self.expert_bytes, self.upload_stream)
            # this pass's residency view: only its experts count as resident for the grouping
            table = np.full(ne, (capi.EMPTY << 32) | SENTINEL, np.uint64)
            for e in batch:
                table[e] = self.cache.entry(e)
            self.upload_stream.synchronize()  # the copy of `table` below reuses pageable memory
            self.pass_table.upload(table)
            uploaded.record(self.upload_stream)
            if compute:
                compute.wait_event(uploaded)
            pf.group_pairs(self.idx, self.w, t, k, ne, self.routes, residency=self.pass_table)
            pf.encode_grouped_expert_gemms(self.pool, self.off, self.routes, hidden, stride, self.partials, self.ffn_ws, t, k)
            served.record(compute)
            (compute.synchronize() if compute else synchronize())
            todo = todo[len(batch):]
            self.passes += 1
        pf.encode_reduce_token_major(self.partials, self.w, self.h2, t, k, d)
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
        from . import host as _host
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
        self.tag = self.tag % 0xFFFF + 1
        full = [1] * 12  # the operators below read only whether a grid's first word is zero
        m.encode_residency_classification(self.idx, self.pool.table, self.hit_count, self.hit_pos, self.miss_count,
                                          self.miss_pos, self.miss_exp, self.resolved, k, ne, full_grids=full,
                                          spec_args=self.spec_args, host_readback=self.readback, tag=self.tag,
                                          topk_weights=self.w, predicted=self.predicted)
        spec = self.spec_args.ptr
        m.encode_spec_phase1(self.pool, self.resolved, self.off, x, self.acts, d, f, k, indirect=spec)
        m.encode_spec_phase2(self.pool, self.resolved, self.off, self.acts, self.w, residual, y, hidden, d, f, k,
                             indirect=spec + 12)
        (compute.synchronize() if compute else synchronize())
        rb = self.readback.array.view(np.uint32)[: 2 + 5 * k].copy()  # counts, experts, weights, hit and miss positions, predictions
        if np.any(rb >> 16 != self.tag):
            raise ShrikeError("router readback carries another launch's tag")  # RouterHostReadback.swift
        rb &= 0xFFFF
        hits, misses = int(rb[0]), int(rb[1])
        experts = rb[2:2 + k].tolist()
        miss_positions = rb[2 + 3 * k: 2 + 3 * k + misses].tolist()
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
        self.tag = self.tag % 0xFFFF + 1
        m.encode_residency_classification(self.idx, self.pool.table, self.hit_count, self.hit_pos, self.miss_count,
                                          self.miss_pos, self.miss_exp, self.resolved, k, ne, full_grids=[1] * 12,
                                          spec_args=self.spec_args, host_readback=self.readback, tag=self.tag,
                                          topk_weights=self.w, predicted=self.predicted)
        spec = self.spec_args.ptr
        m.encode_spec_phase1(self.pool, self.resolved, self.off, x, self.acts, d, f, k, indirect=spec)
        m.encode_spec_phase2(self.pool, self.resolved, self.off, self.acts, self.w, residual, y, hidden, d, f, k,
                             indirect=spec + 12)
        (compute.synchronize() if compute else synchronize())
        rb = self.readback.array.view(np.uint32)[: 2 + 5 * k].copy()
        if np.any(rb >> 16 != self.tag):
            raise ShrikeError("router readback carries another launch's tag")
        rb &= 0xFFFF
        misses = int(rb[1])
        experts = rb[2:2 + k].tolist()
        miss_positions = rb[2 + 3 * k: 2 + 3 * k + misses].tolist()
        self.predicted_next = rb[2 + 4 * k: 2 + 5 * k].tolist() if probe is not None else []

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
