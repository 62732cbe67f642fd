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

    def encode_decode_layer_batch(self, args: DecodeLayerArgs, tokens: int, x_stride: int):
        """The fused layer for `tokens` sequences, one token each (shrike_hip_moe_decode_layer_batch)."""
        check(capi.load().shrike_hip_moe_decode_layer_batch(self.handle, self._s(), C.byref(args), tokens, x_stride),
              "shrike_hip_moe_decode_layer_batch")

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
                     hidden_stride_elements, ffn_workspace=None):
        """ffn_workspace: the grouped FFN's workspace, which then also takes the group sums of `hidden`
        (encode_grouped_expert_gemms(..., presummed=True) uses them instead of forming them again)."""
        if ffn_workspace is not None:
            check(capi.load().shrike_hip_prefill_router_with_group_sums(
                self.moe.handle, self._s(), ptr(weights), ptr(scales), ptr(biases), ptr(hidden), ptr(effective_scale),
                ptr(per_expert_scale), ptr(logit_bias), ptr(out_indices), ptr(out_weights), ptr(logits_workspace),
                query_count, num_experts, d, top_k, hidden_stride_elements, ptr(ffn_workspace)),
                "shrike_hip_prefill_router_with_group_sums")
            return
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
                                    top_k, max_row_tiles=None, presummed=False):
        fn = capi.load().shrike_hip_prefill_grouped_ffn_presummed if presummed else capi.load().shrike_hip_prefill_grouped_ffn
        check(fn(
            self.moe.handle, self._s(), pool.bases, pool.stride, C.byref(offsets), C.byref(routes.c),
            routes.max_row_tiles if max_row_tiles is None else max_row_tiles, ptr(hidden), hidden_stride_elements,
            ptr(route_partials), ptr(workspace), workspace.nbytes, query_count, self.moe.desc.d, self.moe.desc.f, top_k),
            "shrike_hip_prefill_grouped_ffn_presummed" if presummed else "shrike_hip_prefill_grouped_ffn")

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
