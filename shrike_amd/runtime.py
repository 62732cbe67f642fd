"""Thin Python face of the C ABI for tests, the smoke run and the benchmark.

Everything runs through libshrikehip (include/shrike_hip.h): device memory, streams
and events come from its plumbing calls, host arrays are numpy. No other GPU
runtime is loaded, and nothing here computes on the CPU.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import capi
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
    return b.ptr if isinstance(b, DeviceBuffer) else int(b)


class Stream:
    def __init__(self):
        init()
        self.handle = capi.load().shrike_hip_stream_create()
        if not self.handle:
            raise ShrikeError(capi.last_error())

    def synchronize(self):
        check(capi.load().shrike_hip_stream_synchronize(self.handle), "stream_synchronize")

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
