"""Host-side mirror of the reference's prefill bookkeeping and slot cache over the C ABI
(include/shrike_host.h). Names follow the reference's Swift types; every function calls
into libshrikehip.so — nothing here computes a result in Python."""
from __future__ import annotations

import ctypes as C
import os
import errno

import numpy as np

from . import capi
from .capi import ShrikeError

PAIR_DTYPE = np.dtype([("token", "<u4"), ("expert", "<u4"), ("rank", "<u4"), ("weight_bits", "<u4")])
GROUP_DTYPE = np.dtype([("expert", "<u4"), ("pair_start", "<u4"), ("pair_count", "<u4")])
TILE_DTYPE = np.dtype([("group_start", "<u4"), ("group_count", "<u4"), ("pair_start", "<u4"), ("pair_count", "<u4")])
BLOCK_DTYPE = np.dtype([("slot", "<u4"), ("pair_start", "<u4"), ("rows", "<u4"), ("staging_row", "<u4"),
                        ("row_tile_start", "<u4")])
WAVE_DTYPE = np.dtype([("block_start", "<u4"), ("block_count", "<u4"), ("padded_rows", "<u4"), ("tail_rows", "<u4")])

GROUPING_ERRORS = {
    1: "invalidQueryCount", 2: "invalidTopK", 3: "invalidNumExperts", 4: "invalidTileExpertCount",
    5: "pairCountMismatch", 6: "tokenOutOfRange", 7: "rankOutOfRange", 8: "expertOutOfRange",
    9: "duplicateTokenRank", 10: "expertSortKeyCountMismatch",
}
_ERROR_ARITY = {5: 2, 9: 2, 10: 2}


def _vp(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _as(a, struct):
    return a.ctypes.data_as(C.POINTER(struct))


class GroupingError(ShrikeError):
    """PrefillMoEGroupingError (PrefillMoEGrouping.swift:52-89): `case` names the Swift case,
    `values` its associated values."""

    def __init__(self, code, values, message):
        super().__init__(message)
        self.code, self.case = code, GROUPING_ERRORS.get(code, "invalidArgument")
        self.values = tuple(values[: _ERROR_ARITY.get(code, 1)])


class GroupedRoutes:
    """PrefillMoEGroupedRoutes (PrefillMoEGrouping.swift:32-50) as numpy arrays."""

    def __init__(self, sorted_pairs, offsets, counts, groups, tiles, maxima, query_count):
        self.sorted_pairs, self.per_expert_offsets, self.per_expert_counts = sorted_pairs, offsets, counts
        self.groups, self.tiles, self.query_count = groups, tiles, query_count
        self.max_pairs_per_expert, self.max_pairs_per_tile, self.max_live_experts_per_tile = maxima


def make_token_expert_pairs(indices, weights_f16_bits, query_count: int, top_k: int) -> np.ndarray:
    """PrefillRouter.makeTokenExpertPairs (PrefillRouter.swift:160-180)."""
    idx = np.ascontiguousarray(indices, dtype=np.uint32)
    w = np.ascontiguousarray(weights_f16_bits, dtype=np.uint16)
    if idx.size != query_count * top_k or w.size != query_count * top_k:
        raise ShrikeError("indices/weights count mismatch")  # the reference's precondition
    out = np.zeros(query_count * top_k, dtype=PAIR_DTYPE)
    capi.check(capi.load().shrike_make_token_expert_pairs(_vp(idx), _vp(w), query_count, top_k,
                                                          _as(out, capi.TokenExpertPair)), "makeTokenExpertPairs")
    return out


def group_token_expert_pairs(pairs: np.ndarray, query_count: int, top_k: int, num_experts: int,
                             tile_expert_count: int = 16, expert_sort_keys=None) -> GroupedRoutes:
    """PrefillMoEGrouping.groupTokenExpertPairs (PrefillMoEGrouping.swift:269-370)."""
    pairs = np.ascontiguousarray(pairs, dtype=PAIR_DTYPE)
    n, e = pairs.size, max(int(num_experts), 0)
    cap = max(1, min(e, n))
    sorted_pairs = np.zeros(max(n, 1), dtype=PAIR_DTYPE)
    offsets, counts = np.zeros(max(e, 1), np.uint32), np.zeros(max(e, 1), np.uint32)
    groups, tiles = np.zeros(cap, GROUP_DTYPE), np.zeros(cap, TILE_DTYPE)
    out = capi.GroupedRoutes(_as(sorted_pairs, capi.TokenExpertPair), _as(offsets, C.c_uint32), _as(counts, C.c_uint32),
                             _as(groups, capi.MoEGroup), _as(tiles, capi.MoETile))
    keys = None if expert_sort_keys is None else np.ascontiguousarray(expert_sort_keys, dtype=np.uint64)
    rc = capi.load().shrike_group_pairs(_as(pairs, capi.TokenExpertPair), n, query_count, top_k, num_experts,
                                        tile_expert_count, _vp(keys), 0 if keys is None else keys.size, C.byref(out))
    if rc != 0:
        raise GroupingError(rc, list(out.error_value), capi.last_error())
    return GroupedRoutes(sorted_pairs[:n], offsets[:e], counts[:e], groups[: out.group_count], tiles[: out.tile_count],
                         (out.max_pairs_per_expert, out.max_pairs_per_tile, out.max_live_experts_per_tile), query_count)


def resident_first_balanced(rows_by_expert: dict, last_row_by_expert: dict, resident, slots: int,
                            tile_width: int) -> list:
    """PrefillSweepOrder.residentFirstBalanced (PrefillMoEGrouping.swift:131-177)."""
    experts = np.array(list(last_row_by_expert.keys()), dtype=np.uint32)
    rows = np.array([rows_by_expert.get(int(e), 0) for e in experts], dtype=np.int64)
    last = np.array([last_row_by_expert[int(e)] for e in experts], dtype=np.int64)
    res = np.ascontiguousarray(np.asarray(resident, dtype=np.uint8))
    out = np.zeros(max(1, experts.size), np.uint32)
    count = C.c_size_t(0)
    capi.check(capi.load().shrike_sweep_order_resident_first_balanced(
        _vp(experts), _vp(rows), _vp(last), experts.size, _vp(res), res.size, slots, tile_width, _vp(out),
        C.byref(count)), "residentFirstBalanced")
    return out[: count.value].tolist()


def expert_sort_keys(order, num_experts: int) -> np.ndarray:
    """PrefillSweepOrder.expertSortKeys (PrefillMoEGrouping.swift:196-202)."""
    o = np.ascontiguousarray(order, dtype=np.uint32)
    keys = np.zeros(max(1, num_experts), np.uint64)
    capi.load().shrike_expert_sort_keys(_vp(o), o.size, num_experts, _vp(keys))
    return keys[:num_experts]


class PlanError(ShrikeError):
    pass


def plan_expert_waves(ranges, bound_experts, staging_rows: int, row_tile: int = 64, tail_tile: int = 0):
    """PrefillGroupedRoutedMoE.planExpertWaves (PrefillGroupedRoutedMoE.swift:104-241).
    `ranges`: (expert, pair_start, pair_count). Returns (blocks, waves) structured arrays."""
    r = (capi.ExpertPairRange * max(1, len(ranges)))(*[capi.ExpertPairRange(*x) for x in ranges])
    bound = np.ascontiguousarray(bound_experts, dtype=np.uint32)
    lib = capi.load()
    cap_b, cap_w = 64, 16
    while True:
        blocks, waves = np.zeros(cap_b, BLOCK_DTYPE), np.zeros(cap_w, WAVE_DTYPE)
        nb, nw = C.c_size_t(0), C.c_size_t(0)
        rc = lib.shrike_plan_expert_waves(r, len(ranges), _vp(bound), bound.size, staging_rows, row_tile, tail_tile,
                                          _as(blocks, capi.RoutedExpertBlock), cap_b, C.byref(nb),
                                          _as(waves, capi.RoutedExpertWave), cap_w, C.byref(nw))
        if rc == errno.ENOSPC:
            cap_b, cap_w = max(cap_b, nb.value), max(cap_w, nw.value)
            continue
        if rc != 0:
            raise PlanError(capi.last_error())
        return blocks[: nb.value], waves[: nw.value]


def row_tile_table(blocks: np.ndarray, wave, row_tile: int = 64) -> list:
    """rowTileTable (PrefillGroupedRoutedMoE.swift:272-283) for one wave of `blocks`."""
    b = np.ascontiguousarray(blocks[int(wave["block_start"]): int(wave["block_start"]) + int(wave["block_count"])])
    table = np.zeros(max(1, int(wave["padded_rows"]) // row_tile), np.uint32)
    capi.check(capi.load().shrike_row_tile_table(_as(b, capi.RoutedExpertBlock), b.size, int(wave["padded_rows"]),
                                                 row_tile, _vp(table)), "rowTileTable")
    return table[: int(wave["padded_rows"]) // row_tile].tolist()


def row_tile_tables(blocks: np.ndarray, wave):
    """rowTileTables (PrefillGroupedRoutedMoE.swift:247-269): (gather, body, tail)."""
    b = np.ascontiguousarray(blocks[int(wave["block_start"]): int(wave["block_start"]) + int(wave["block_count"])])
    padded, tail_rows = int(wave["padded_rows"]), int(wave["tail_rows"])
    ng, nb, nt = padded // 32, (padded - tail_rows) // 64, tail_rows // 32
    g, bo, t = (np.zeros(max(1, n), np.uint32) for n in (ng, nb, nt))
    capi.check(capi.load().shrike_row_tile_tables(_as(b, capi.RoutedExpertBlock), b.size, padded, tail_rows,
                                                  _vp(g), _vp(bo), _vp(t)), "rowTileTables")
    return g[:ng].tolist(), bo[:nb].tolist(), t[:nt].tolist()


class CachePlan:
    """ExpertCachePlan (PreadExpertStreamer.swift:17-38)."""

    def __init__(self, n: int):
        self.experts_a = np.zeros(max(1, n), np.int32)
        self.slots_a = np.zeros(max(1, n), np.int32)
        self.gens_a = np.zeros(max(1, n), np.uint64)
        self.misses_a = np.zeros(max(1, n), np.uint32)
        self.cells_a = np.zeros(max(1, n), np.uint32)
        self.adopted_a = np.zeros(max(1, n), np.uint32)
        self.freed_experts_a = np.zeros(max(1, n), np.int32)
        self.freed_cells_a = np.zeros(max(1, n), np.uint32)
        self.c = capi.ExpertCachePlan(0, 0, _as(self.experts_a, C.c_int32), _as(self.slots_a, C.c_int32),
                                      _as(self.gens_a, C.c_uint64), _as(self.misses_a, C.c_uint32), 0, 0,
                                      _as(self.cells_a, C.c_uint32), _as(self.adopted_a, C.c_uint32), 0, 0,
                                      _as(self.freed_experts_a, C.c_int32), _as(self.freed_cells_a, C.c_uint32))

    @property
    def experts(self):
        return self.experts_a[: self.c.expert_count].tolist()

    @property
    def assigned_slots(self):
        return self.slots_a[: self.c.expert_count].tolist()

    @property
    def assigned_generations(self):
        return self.gens_a[: self.c.expert_count].tolist()

    @property
    def misses(self):
        return self.misses_a[: self.c.miss_count].tolist()

    @property
    def hits(self):
        return self.c.hits

    @property
    def layer(self):
        return self.c.layer

    @property
    def assigned_cells(self):
        """The arena cell behind each assigned slot (what expertCachePlanBuffers binds)."""
        return self.cells_a[: self.c.expert_count].tolist()

    @property
    def adopted(self):
        return self.adopted_a[: self.c.adopted_count].tolist()

    @property
    def freed_cells(self):
        """freedCells: expert -> the pool cell its landing's swap gave back to the ring."""
        n = self.c.freed_count
        return dict(zip(self.freed_experts_a[:n].tolist(), self.freed_cells_a[:n].tolist()))


class CellArena:
    """ExpertCellArena's numbering and generations (ExpertCellArena.swift:16-29, :95-104); the cells' bytes
    belong to the HBM pool."""

    def __init__(self, cell_count: int):
        err = C.c_int(0)
        self._h = capi.load().shrike_cell_arena_create(cell_count, C.byref(err))
        if not self._h:
            raise ShrikeError(f"cell arena: {capi.last_error()}")
        self.cell_count = cell_count

    def cell_generation(self, cell: int) -> int:
        if not 0 <= cell < self.cell_count:
            raise IndexError("expert cell out of range")
        return int(capi.load().shrike_cell_arena_generation(self._h, cell))

    def close(self):
        if self._h:
            capi.load().shrike_cell_arena_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class SlotCache:
    """The slot bookkeeping of PreadExpertStreamer (PreadExpertStreamer.swift:405-543, :676-767)."""

    def __init__(self, slot_count: int, experts_per_layer: int, first_cell: int = 0, slru_share=None,
                 arena: "CellArena | None" = None):
        err = C.c_int(0)
        self.slot_count, self.experts_per_layer = slot_count, experts_per_layer
        self.arena = arena  # kept alive for as long as the cache
        policy = (0 if slru_share is None else 1, 0.0 if slru_share is None else float(slru_share))
        if arena is None:
            self._h = capi.load().shrike_slot_cache_create(slot_count, experts_per_layer, first_cell, *policy,
                                                           C.byref(err))
        else:
            self._h = capi.load().shrike_slot_cache_create_in_arena(arena._h, slot_count, experts_per_layer, first_cell,
                                                                    *policy, C.byref(err))
        if not self._h:
            raise ShrikeError(f"slot cache: {capi.last_error()}")

    def close(self):
        if self._h:
            capi.load().shrike_slot_cache_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def plan(self, experts, layer=0, avoiding_slots=(), protected_experts=None, misses_counted=None,
             gpu_missed_experts=None, leased_landings=()):
        """planExpertsCachedIfPossible: None when the experts cannot be placed."""
        e = np.ascontiguousarray(experts, dtype=np.int32)
        avoid = np.ascontiguousarray(sorted(avoiding_slots), dtype=np.int32)
        prot = None if protected_experts is None else np.ascontiguousarray(np.asarray(protected_experts, dtype=np.uint8))
        missed = np.ascontiguousarray(sorted(gpu_missed_experts or ()), dtype=np.int32)
        leased = np.ascontiguousarray(sorted(leased_landings), dtype=np.int32)
        plan = CachePlan(e.size)
        rc = capi.load().shrike_slot_cache_plan_with_landings(
            self._h, _vp(e), e.size, layer, _vp(avoid) if avoid.size else None, avoid.size, _vp(prot),
            0 if prot is None else prot.size, _vp(missed) if missed.size else None, missed.size,
            _vp(leased) if leased.size else None, leased.size, -1 if misses_counted is None else misses_counted,
            C.byref(plan.c))
        if rc == errno.ENOSPC:
            return None
        capi.check(rc, "planExpertsCached")
        return plan

    def complete(self, plan: CachePlan, elapsed_nanos: int = 0, fetch_nanos: int = 0):
        capi.check(capi.load().shrike_slot_cache_complete(self._h, C.byref(plan.c), elapsed_nanos, fetch_nanos),
                   "markPlanMissesResident")

    def abandon(self, plan: CachePlan):
        capi.load().shrike_slot_cache_abandon(self._h, C.byref(plan.c))

    def load(self, experts, **kw):
        """loadExpertsCached without the reads: plan, then mark the misses resident."""
        plan = self.plan(experts, **kw)
        if plan is None:
            raise ShrikeError(capi.last_error())  # ModelError.expertCacheUnplaceable
        self.complete(plan)
        return plan

    def pin(self, plan: CachePlan):
        capi.check(capi.load().shrike_slot_cache_pin(self._h, C.byref(plan.c)), "pin")

    def unpin(self, slots, generations):
        s, g = np.ascontiguousarray(slots, np.int32), np.ascontiguousarray(generations, np.uint64)
        capi.load().shrike_slot_cache_unpin(self._h, _vp(s), _vp(g), s.size)

    def slot_cell(self, slot: int) -> int:
        """The arena cell behind a slot (cellIndexUnlocked, PreadExpertStreamer.swift:1135-1137)."""
        return int(capi.load().shrike_slot_cache_slot_cell(self._h, slot))

    def owns_cell(self, cell: int) -> bool:
        return bool(capi.load().shrike_slot_cache_owns_cell(self._h, cell))

    def claim_landing(self, expert: int, cell: int) -> bool:
        """claimLanding, PreadExpertStreamer.swift:815-829."""
        return bool(capi.load().shrike_slot_cache_claim_landing(self._h, expert, cell))

    def complete_landing(self, expert: int, cell: int) -> bool:
        """completeLanding, PreadExpertStreamer.swift:834-848."""
        return bool(capi.load().shrike_slot_cache_complete_landing(self._h, expert, cell))

    def fail_landing(self, expert: int, cell: int):
        capi.load().shrike_slot_cache_fail_landing(self._h, expert, cell)

    def drop_landing(self, expert: int, cell: int):
        """dropLanding, PreadExpertStreamer.swift:1010-1018."""
        capi.load().shrike_slot_cache_drop_landing(self._h, expert, cell)

    def claim_prefetch(self, experts, cells):
        """The claims of beginPrefetch (PreadExpertStreamer.swift:1034-1057): raises PrefetchClaimRefused when the
        pool holds a predicted expert, ShrikeError for a cell the pool owns or an expert out of range."""
        if len(experts) != len(cells):
            raise ShrikeError("prefetch experts and cells differ in count")
        e, c = np.ascontiguousarray(experts, np.int32), np.ascontiguousarray(cells, np.int64)
        refused = C.c_uint32(0)
        rc = capi.load().shrike_slot_cache_claim_prefetch(self._h, _vp(e), _vp(c), e.size, C.byref(refused))
        if rc == PREFETCH_CLAIM_REFUSED:
            raise PrefetchClaimRefused(int(e[refused.value]), int(c[refused.value]))
        capi.check(rc, "beginPrefetch")

    def reserve_overflow_slot(self, expert: int, protecting=()):
        """reserveOverflowSlot, PreadExpertStreamer.swift:860-893: the cell, or None."""
        p = np.ascontiguousarray(list(protecting), np.int32)
        cell = capi.load().shrike_slot_cache_reserve_overflow_slot(self._h, expert, _vp(p) if p.size else None, p.size)
        return None if cell < 0 else int(cell)

    def mark_overflow_resident(self, expert: int, cell: int):
        capi.load().shrike_slot_cache_mark_overflow_resident(self._h, expert, cell)

    def abandon_overflow_slot(self, expert: int, cell: int):
        """abandonOverflowSlot, PreadExpertStreamer.swift:980-993."""
        capi.load().shrike_slot_cache_abandon_overflow_slot(self._h, expert, cell)

    def finish_agreed_reads(self, experts, cells, succeeded: bool, elapsed_nanos: int = 0, fetch_nanos: int = 0):
        """The completion of beginAgreedReads (PreadExpertStreamer.swift:936-964)."""
        if len(experts) != len(cells):
            raise ShrikeError("agreed reads' experts and cells differ in count")
        e, c = np.ascontiguousarray(experts, np.int32), np.ascontiguousarray(cells, np.int64)
        capi.check(capi.load().shrike_slot_cache_finish_agreed_reads(self._h, _vp(e), _vp(c), e.size, int(succeeded),
                                                                     elapsed_nanos, fetch_nanos), "beginAgreedReads")

    def statistics(self, expert_stride_bytes: int = 0) -> capi.StreamingStatistics:
        st = capi.StreamingStatistics()
        capi.load().shrike_slot_cache_statistics(self._h, expert_stride_bytes, C.byref(st))
        return st

    def resident_experts(self) -> list:
        out = np.zeros(max(1, self.slot_count), np.int32)
        n = capi.load().shrike_slot_cache_resident_experts(self._h, _vp(out), out.size)
        return out[:n].tolist()

    def entry(self, expert: int) -> int:
        return int(capi.load().shrike_slot_cache_entry(self._h, expert))

    def drain_publications(self):
        e, w = np.zeros(max(1, self.experts_per_layer), np.uint32), np.zeros(max(1, self.experts_per_layer), np.uint64)
        n = capi.load().shrike_slot_cache_drain_publications(self._h, _vp(e), _vp(w), e.size)
        return list(zip(e[:n].tolist(), w[:n].tolist()))


# --------------------------------------------------------------- parallel expert reader

class ReadFailed(ShrikeError):
    """ParallelExpertReader.Failure (sources/Shrike/Infrastructure/Streaming/ParallelExpertReader.swift)."""

    def __init__(self, errno_: int, what: str):
        super().__init__(f"{what}: {os.strerror(errno_)} (errno {errno_})")
        self.errno = errno_


class ParallelExpertReader:
    """shrike_expert_reader with the reference wrapper's names: `threads` workers with a descriptor each,
    up to `batch_depth` batches published at once, pread only."""

    def __init__(self, path: str, expert_stride: int, threads: int = 4, batch_depth: int = 1,
                 bypass_cache: bool = False):
        err = C.c_int(0)
        self.handle = capi.load().shrike_expert_reader_create(os.fsencode(path), expert_stride, threads, batch_depth,
                                                              int(bypass_cache), C.byref(err))
        if not self.handle:
            raise ReadFailed(err.value, f"cannot open {path}")
        self.expert_stride = expert_stride

    def close(self):
        if self.handle:
            capi.load().shrike_expert_reader_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def thread_count(self) -> int:
        return capi.load().shrike_expert_reader_threads(self.handle)

    @property
    def batch_depth(self) -> int:
        return capi.load().shrike_expert_reader_batch_depth(self.handle)

    @staticmethod
    def _destinations(into):
        return (C.c_void_p * len(into))(*[int(p) for p in into])

    def fetch(self, experts, into) -> None:
        """experts[i] * stride -> the address into[i] (each expert_stride bytes long)."""
        if len(experts) != len(into):
            raise ValueError("one destination per expert")
        ids = (C.c_uint32 * len(experts))(*experts)
        rc = capi.load().shrike_expert_reader_fetch(self.handle, ids, self._destinations(into), len(experts))
        if rc:
            raise ReadFailed(rc, "expert read failed")

    def fetch_offsets(self, offsets, into) -> None:
        if len(offsets) != len(into):
            raise ValueError("one destination per offset")
        offs = (C.c_uint64 * len(offsets))(*offsets)
        rc = capi.load().shrike_expert_reader_fetch_offsets(self.handle, offs, self._destinations(into), len(offsets))
        if rc:
            raise ReadFailed(rc, "expert read failed")


# --------------------------------------------------------------- packed experts layout

class LayoutError(ShrikeError):
    """ModelError.indexCorrupt / .missingFile of the layout reader, with the library's errno."""

    def __init__(self, errno_: int, message: str):
        super().__init__(message)
        self.errno = errno_


class PackedExpertsLayout:
    """packed_experts/layout.json (sources/Shrike/Infrastructure/ModelIO/PackedExpertsLayout.swift:34-129)."""

    def __init__(self, handle):
        self.handle = handle

    @staticmethod
    def _made(handle, err):
        if not handle:
            raise LayoutError(err.value, capi.load().shrike_host_last_error().decode())
        return PackedExpertsLayout(handle)

    @classmethod
    def decode(cls, data: bytes) -> "PackedExpertsLayout":
        err = C.c_int(0)
        return cls._made(capi.load().shrike_packed_layout_decode(data, len(data), C.byref(err)), err)

    @classmethod
    def load(cls, model_dir: str, max_bytes: int = 0) -> "PackedExpertsLayout":
        err = C.c_int(0)
        return cls._made(capi.load().shrike_packed_layout_load(os.fsencode(model_dir), max_bytes, C.byref(err)), err)

    def close(self):
        if self.handle:
            capi.load().shrike_packed_layout_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def expert_stride(self) -> int:
        return capi.load().shrike_packed_layout_expert_stride(self.handle)

    @property
    def num_layers(self) -> int:
        return capi.load().shrike_packed_layout_num_layers(self.handle)

    @property
    def experts_per_layer(self) -> int:
        return capi.load().shrike_packed_layout_experts_per_layer(self.handle)

    def _check(self, rc):
        if rc:
            raise LayoutError(rc, capi.load().shrike_host_last_error().decode())

    def layer(self, index: int) -> dict:
        lid, file, count = C.c_int(0), C.c_char_p(), C.c_int(0)
        self._check(capi.load().shrike_packed_layout_layer(self.handle, index, C.byref(lid), C.byref(file), C.byref(count)))
        return {"layer": lid.value, "file": file.value.decode(), "expert_count": count.value}

    def expert(self, layer: int, expert: int) -> dict:
        out = capi.PackedExpert()
        self._check(capi.load().shrike_packed_layout_expert(self.handle, layer, expert, C.byref(out)))
        return {"expert": out.expert, "physical_rank": out.physical_rank, "offset": out.offset, "size": out.size,
                "tensor_count": out.tensor_count}

    def tensor(self, layer: int, expert: int, role: str):
        out = capi.PackedTensor()
        rc = capi.load().shrike_packed_layout_tensor(self.handle, layer, expert, role.encode(), C.byref(out))
        if rc == 2:  # ENOENT: the blob has no such sub-tensor
            return None
        self._check(rc)
        return {"offset": out.offset, "size": out.size, "dtype": out.dtype.decode(),
                "shape": [out.shape[i] for i in range(min(out.rank, 4))], "bits": out.bits or None}

    def expert_offsets(self, layer: int, additive_biases: bool = False) -> capi.ExpertOffsets:
        out = capi.ExpertOffsets()
        self._check(capi.load().shrike_packed_layout_expert_offsets(self.handle, layer, int(additive_biases), C.byref(out)))
        return out

    def cross_validate(self, num_layers: int, experts_per_layer: int, expert_stride: int, file_sizes: dict) -> None:
        paths = (C.c_char_p * len(file_sizes))(*[k.encode() for k in file_sizes])
        sizes = (C.c_uint64 * len(file_sizes))(*file_sizes.values())
        self._check(capi.load().shrike_packed_layout_cross_validate(self.handle, num_layers, experts_per_layer,
                                                                    expert_stride, paths, sizes, len(file_sizes)))


# --------------------------------------------------------------- routed tile loop of a streamed prefill chunk

ISSUE_WITHOUT_PENDING, PREFETCH_NEXT, DRAIN_NO_ASSIGNED_SLOTS, DRAIN_PLAN_UNAVAILABLE, DRAIN_MAX_DEPTH = range(5)
BATCH_OPEN, BATCH_FULL, BATCH_LAST_TILE = range(3)


class TileSchedulerConfig:
    """PrefillRoutedTileSchedulerConfig (PrefillRoutedTileScheduler.swift:46-96); the constructor clamps."""

    def __init__(self, max_pending_depth=1, tile_experts=8, tiles_per_command_buffer=1, fetch_lookahead=0):
        self.c = capi.TileSchedulerConfig()
        capi.load().shrike_tile_scheduler_config_make(max_pending_depth, tile_experts, tiles_per_command_buffer,
                                                      fetch_lookahead, C.byref(self.c))

    def astuple(self):
        return (self.c.max_pending_depth, self.c.tile_experts, self.c.tiles_per_command_buffer, self.c.fetch_lookahead)

    max_pending_depth = property(lambda self: self.c.max_pending_depth)
    tile_experts = property(lambda self: self.c.tile_experts)
    tiles_per_command_buffer = property(lambda self: self.c.tiles_per_command_buffer)
    fetch_lookahead = property(lambda self: self.c.fetch_lookahead)

    def __eq__(self, other):
        return isinstance(other, TileSchedulerConfig) and self.astuple() == other.astuple()

    def __repr__(self):
        return "TileSchedulerConfig(depth=%d, experts=%d, width=%d, lookahead=%d)" % self.astuple()

    def fits_slot_budget(self, slot_count: int, reserved_hits: int = 0) -> bool:
        return bool(capi.load().shrike_tile_scheduler_fits_slot_budget(C.byref(self.c), slot_count, reserved_hits))

    def fitting(self, slot_count: int, reserved_hits: int = 0):
        out = TileSchedulerConfig()
        if not capi.load().shrike_tile_scheduler_fitting(C.byref(self.c), slot_count, reserved_hits, C.byref(out.c)):
            return None
        return out


class TileScheduler:
    """PrefillRoutedTileScheduler (PrefillRoutedTileScheduler.swift:98-156)."""

    def __init__(self, config: TileSchedulerConfig | None = None):
        self.config = config or TileSchedulerConfig()

    def decide(self, has_pending_tile: bool, pending_assigned_slots, avoiding_slot_plan_available: bool, pending_depth=None):
        """The decision code; for PREFETCH_NEXT the slots to avoid are pending_assigned_slots as given."""
        return capi.load().shrike_tile_scheduler_decide(C.byref(self.config.c), int(has_pending_tile),
                                                        -1 if pending_depth is None else pending_depth,
                                                        len(pending_assigned_slots), int(avoiding_slot_plan_available))

    def plans_lookahead(self, index: int, tile_count: int) -> bool:
        return bool(capi.load().shrike_tile_scheduler_plans_lookahead(C.byref(self.config.c), index, tile_count))

    def should_begin_lookahead(self, index: int, tile_count: int, avoiding_slot_plan_available: bool) -> bool:
        return bool(capi.load().shrike_tile_scheduler_should_begin_lookahead(C.byref(self.config.c), index, tile_count,
                                                                             int(avoiding_slot_plan_available)))

    def batch_action(self, open_batch_tiles: int, open_batch_slots, next_tile_plan_available: bool, is_last_tile: bool):
        out = capi.TileBatchAction()
        capi.load().shrike_tile_scheduler_batch_action(C.byref(self.config.c), open_batch_tiles, len(open_batch_slots),
                                                       int(next_tile_plan_available), int(is_last_tile), C.byref(out))
        return bool(out.commit_before_append), out.commit_after_append


class TileSequencer:
    """PrefillRoutedTileSequencer.run over a Python driver object with the protocol's members
    (PrefillRoutedTileSequencer.swift:3-24): properties open_batch_tiles, open_batch_slots, pending_depth,
    pending_assigned_slots; methods plan(tile, avoiding_in_flight) -> bool, begin, abandon_plan, encode,
    commit_open_batch, drain_oldest_batch, abandon_begun_fetches. An exception raised by the driver ends the
    run, reaches abandon_begun_fetches first and is raised again from run()."""

    def __init__(self, scheduler: TileScheduler):
        self.scheduler = scheduler

    def run(self, tile_count: int, driver) -> None:
        raised = []

        def guarded(fn):
            def call(_ctx, *args):
                try:
                    fn(*args)
                    return 0
                except BaseException as exc:  # noqa: BLE001 - carried across the C frame
                    raised.append(exc)
                    return errno.ECANCELED
            return call

        def plan(_ctx, tile, avoiding, available):
            try:
                available[0] = int(bool(driver.plan(tile, None if avoiding < 0 else avoiding)))
                return 0
            except BaseException as exc:  # noqa: BLE001
                raised.append(exc)
                return errno.ECANCELED

        T = capi.TileDriver
        fields = dict(T._fields_)
        d = T(None,
              fields["open_batch_tiles"](lambda _c: driver.open_batch_tiles),
              fields["open_batch_slot_count"](lambda _c: len(driver.open_batch_slots)),
              fields["pending_depth"](lambda _c: driver.pending_depth),
              fields["pending_assigned_slot_count"](lambda _c: len(driver.pending_assigned_slots)),
              fields["plan"](plan),
              fields["begin"](guarded(driver.begin)),
              fields["abandon_plan"](guarded(driver.abandon_plan)),
              fields["encode"](guarded(driver.encode)),
              fields["commit_open_batch"](lambda _c: driver.commit_open_batch()),
              fields["drain_oldest_batch"](guarded(driver.drain_oldest_batch)),
              fields["abandon_begun_fetches"](lambda _c: driver.abandon_begun_fetches()))
        rc = capi.load().shrike_tile_sequencer_run(C.byref(self.scheduler.config.c), tile_count, C.byref(d))
        if raised:
            raise raised[0]
        if rc:
            raise ShrikeError(f"tile sequencer failed with {rc}: {capi.last_error()}")


class ChunkExpertProtection:
    """PrefillChunkExpertProtection (RealForwardRunner.swift:63-93)."""

    def __init__(self, routed_experts, experts_per_layer: int):
        self._r = (C.c_uint8 * experts_per_layer)()
        ids = (C.c_int32 * len(routed_experts))(*routed_experts)
        capi.load().shrike_chunk_protection_init(ids, len(routed_experts), self._r, experts_per_layer)

    @property
    def remaining(self):
        return [bool(v) for v in self._r]

    def planning(self, tile_experts) -> None:
        ids = (C.c_int32 * len(tile_experts))(*tile_experts)
        capi.load().shrike_chunk_protection_planning(ids, len(tile_experts), self._r, len(self._r))


class TileLifetimeError(ShrikeError):
    """PrefillStreamedTileLifetimeError (PrefillGroupedRoutedMoE.swift:376-386)."""

    def __init__(self, code, conflicting_tile, message):
        super().__init__(message)
        self.code, self.conflicting_tile = code, conflicting_tile


class TileSlotLifetime:
    """PrefillStreamedTileSlotLifetime (PrefillGroupedRoutedMoE.swift:388-424)."""

    def __init__(self):
        self._h = capi.load().shrike_tile_lifetime_create()

    def __del__(self):
        try:
            if self._h:
                capi.load().shrike_tile_lifetime_destroy(self._h)
                self._h = None
        except Exception:
            pass

    def begin(self, tile_index: int, planned_slots) -> None:
        slots = (C.c_int32 * len(planned_slots))(*planned_slots)
        other = C.c_int(-1)
        rc = capi.load().shrike_tile_lifetime_begin(self._h, tile_index, slots, len(planned_slots), C.byref(other))
        if rc:
            raise TileLifetimeError(rc, other.value, capi.last_error())

    def complete(self, tile_index: int) -> None:
        rc = capi.load().shrike_tile_lifetime_complete(self._h, tile_index)
        if rc:
            raise TileLifetimeError(rc, -1, capi.last_error())


# ------------------------------------------------------------------ load operations and the prefetch ring

LOAD_SUBMITTED, LOAD_IN_FLIGHT, LOAD_COMPLETED, LOAD_FAILED = 0, 1, 2, 3
PREFETCH_CLAIM_REFUSED = -2


def monotonic_nanos() -> int:
    return int(capi.load().shrike_monotonic_nanos())


class ExpertLoadOperation:
    """ExpertLoadOperation (sources/Shrike/Infrastructure/Streaming/ExpertLoadOperation.swift:15-153): one
    storage batch, submitted now and finished later by whoever reads it."""

    def __init__(self):
        self._h = capi.load().shrike_load_operation_create()
        if not self._h:
            raise MemoryError("load operation")

    def __del__(self):
        try:
            if self._h:
                capi.load().shrike_load_operation_release(self._h)
                self._h = None
        except Exception:
            pass

    @property
    def state(self) -> int:
        return capi.load().shrike_load_operation_state(self._h)

    def mark_in_flight(self) -> None:
        rc = capi.load().shrike_load_operation_mark_in_flight(self._h)
        if rc:
            raise ShrikeError(f"expert load operation started more than once (code {rc})")

    def finish(self, failure: int = 0) -> None:
        rc = capi.load().shrike_load_operation_finish(self._h, failure)
        if rc:
            raise ShrikeError(f"expert load operation completed more than once (code {rc})")

    def wait(self) -> None:
        rc = capi.load().shrike_load_operation_wait(self._h)
        if rc:
            raise ReadFailed(rc, "expert load operation")

    def wait_until(self, deadline_nanos: int) -> bool:
        return bool(capi.load().shrike_load_operation_wait_until(self._h, deadline_nanos))

    @property
    def submitted_nanos(self) -> int:
        return int(capi.load().shrike_load_operation_submitted_nanos(self._h))

    @property
    def started_nanos(self) -> int:
        return int(capi.load().shrike_load_operation_started_nanos(self._h))

    @property
    def completed_nanos(self) -> int:
        return int(capi.load().shrike_load_operation_completed_nanos(self._h))


class PrefetchClaimRefused(Exception):
    """PrefetchClaimRefused (PreadExpertStreamer.swift:46-49): the pool already holds a predicted expert."""

    def __init__(self, expert: int = -1, cell: int = -1):
        super().__init__(f"prefetch claim refused: expert {expert}, cell {cell}")
        self.expert, self.cell = expert, cell


class ExpertIOScheduler:
    """ExpertIOScheduler (sources/Shrike/Infrastructure/Streaming/ExpertLoadOperation.swift:166-219): the library's
    submission threads (shrike_io_scheduler_*); a queued demand batch runs before any queued speculative one. A
    submitted callable is kept alive until it has run."""

    DEMAND, SPECULATIVE = 0, 1

    def __init__(self, worker_count: int = 4):
        import threading
        if worker_count <= 0:
            raise ValueError("workerCount must be positive")
        err = C.c_int(0)
        self._h = capi.load().shrike_io_scheduler_create(worker_count, C.byref(err))
        if not self._h:
            raise ShrikeError(capi.last_error())
        self._lock = threading.Lock()
        self._pending = {}
        self._next = 1

        def run(context):
            with self._lock:
                work = self._pending.pop(context)
            work()
        self._trampoline = capi.IO_WORK(run)  # one C callback for every submission; the context word names the work

    def submit(self, work, priority: int = 0) -> None:
        with self._lock:
            key, self._next = self._next, self._next + 1
            self._pending[key] = work
        rc = capi.load().shrike_io_scheduler_submit(self._h, priority, self._trampoline, key)
        if rc != 0:
            with self._lock:
                self._pending.pop(key, None)
            raise ShrikeError(capi.last_error())

    def close(self) -> None:
        """Runs what is queued, then ends the threads."""
        if self._h:
            capi.load().shrike_io_scheduler_close(self._h)

    def __del__(self):
        try:
            if self._h:
                capi.load().shrike_io_scheduler_destroy(self._h)
                self._h = None
        except Exception:
            pass


class ExpertIOTimeline:
    """ExpertIOEventCoordinator (sources/Shrike/Infrastructure/Streaming/ExpertIOEventCoordinator.swift:23-90):
    values never reused, status words in a ring, the published value held behind an out-of-order completion."""

    def __init__(self, status_words: int | None = None, word_count: int = 0):
        err = C.c_int(0)
        self._h = capi.load().shrike_io_timeline_create(status_words, word_count, C.byref(err))
        if not self._h:
            raise ShrikeError(capi.last_error())

    def reserve(self) -> "capi.IOCompletionToken":
        token = capi.IOCompletionToken()
        if capi.load().shrike_io_timeline_reserve(self._h, C.byref(token)) != 0:
            raise ShrikeError(capi.last_error())
        return token

    def publish(self, token, succeeded: bool) -> int:
        return int(capi.load().shrike_io_timeline_publish(self._h, C.byref(token), int(bool(succeeded))))

    @property
    def published(self) -> int:
        return int(capi.load().shrike_io_timeline_published(self._h))

    def __del__(self):
        try:
            if self._h:
                capi.load().shrike_io_timeline_destroy(self._h)
                self._h = None
        except Exception:
            pass


class RouterHostReadback:
    """RouterHostReadback (sources/Shrike/Runtime/Inference/RouterHostReadback.swift:8-63) over the library's
    shrike_router_readback_*: `words` is the address of the tagged words (pinned host memory a kernel writes)."""

    @staticmethod
    def word_count(top_k: int) -> int:
        return int(capi.load().shrike_router_readback_word_count(top_k))

    @staticmethod
    def word(tag: int, value: int) -> int:
        return int(capi.load().shrike_router_readback_word(tag, value))

    @staticmethod
    def next_tag(tag: int) -> int:
        return int(capi.load().shrike_router_readback_next_tag(tag))

    @staticmethod
    def is_complete(words: int, top_k: int, tag: int) -> bool:
        return bool(capi.load().shrike_router_readback_is_complete(words, top_k, tag))

    @staticmethod
    def _fields(r, top_k):
        return dict(hit_count=int(r.hit_count), miss_count=int(r.miss_count), expert_ids=list(r.expert_ids[:top_k]),
                    weight_bits=list(r.weight_bits[:top_k]), hit_positions=list(r.hit_positions[:r.hit_count]),
                    miss_positions=list(r.miss_positions[:r.miss_count]), predicted_ids=list(r.predicted_ids[:top_k]))

    @classmethod
    def decode(cls, words: int, top_k: int, tag: int):
        r = capi.RouterReadback()
        if not capi.load().shrike_router_readback_decode(words, top_k, tag, C.byref(r)):
            return None
        return cls._fields(r, top_k)

    @classmethod
    def poll(cls, words: int, top_k: int, tag: int, timeout_nanos: int):
        """Polls the words until every one carries the tag (the command may still be running); None at the deadline."""
        r = capi.RouterReadback()
        if not capi.load().shrike_router_readback_poll(words, top_k, tag, monotonic_nanos() + timeout_nanos, C.byref(r)):
            return None
        return cls._fields(r, top_k)


def int4_affine_gemv(weights: np.ndarray, scales: np.ndarray, biases: np.ndarray, x: np.ndarray, rows: int, n: int) -> np.ndarray:
    """shrike_int4_affine_gemv (sources/ShrikeKernelsC/include/shrike_kernels.h:23-29) on host arrays."""
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(rows, np.float32)
    capi.load().shrike_int4_affine_gemv(weights.ctypes.data, scales.ctypes.data, biases.ctypes.data, x.ctypes.data, rows, n,
                                        out.ctypes.data)
    return out


def cpu_expert_ffn_accumulate(blob: np.ndarray, offsets, x: np.ndarray, d: int, f: int, route_weight: float, out: np.ndarray,
                              scratch: np.ndarray | None = None) -> np.ndarray:
    """CPUExpertFFN.accumulate (sources/Shrike/Kernels/CPU/CPUExpertFFN.swift:102-140): out += w * FFN(x), fp32."""
    L = capi.load()
    if scratch is None:
        scratch = np.empty(L.shrike_cpu_expert_ffn_scratch_floats(d, f), np.float32)
    x = np.ascontiguousarray(x, np.float32)
    rc = L.shrike_cpu_expert_ffn_accumulate(blob.ctypes.data, C.byref(offsets), x.ctypes.data, d, f, route_weight,
                                            scratch.ctypes.data, out.ctypes.data)
    if rc != 0:
        raise ShrikeError(capi.last_error())
    return out


def _ints(values):
    values = list(values)
    return (C.c_int * max(1, len(values)))(*values), len(values)


class ExpertPrefetchRing:
    """ExpertPrefetchRing (sources/Shrike/Runtime/Inference/ExpertPrefetchRing.swift:42-352). `drop(layer, expert,
    cell)` is called with the ring locked. `issue(experts, cells)` passed to begin returns the batch's
    ExpertLoadOperation, raises PrefetchClaimRefused (counted, not propagated) or anything else
    (propagated after the slots are rolled back)."""

    _ISSUE_FAILED = 5  # EIO: the code that carries a Python exception across the C boundary

    def __init__(self, cells, drop=None):
        self._drop = drop or (lambda layer, expert, cell: None)
        self._drop_c = capi.PREFETCH_DROP(lambda _ctx, layer, expert, cell: self._drop(layer, expert, cell))
        arr, n = _ints(cells)
        err = C.c_int(0)
        self._h = capi.load().shrike_prefetch_ring_create(arr, n, self._drop_c, None, C.byref(err))
        if not self._h:
            raise ShrikeError("invalid prefetch ring geometry")  # ExpertPrefetchRing.swift:96-98

    def __del__(self):
        try:
            if self._h:
                capi.load().shrike_prefetch_ring_destroy(self._h)
                self._h = None
        except Exception:
            pass

    def begin(self, layer: int, experts, resident=(), deferred: bool = False, issue=None) -> None:
        raised = []

        def trampoline(_ctx, c_experts, c_cells, count, out_operation):
            try:
                operation = issue([c_experts[i] for i in range(count)], [c_cells[i] for i in range(count)])
                out_operation[0] = operation._h
                raised.append(operation)  # keeps the caller's reference alive until the ring holds its own
                return 0
            except PrefetchClaimRefused:
                return PREFETCH_CLAIM_REFUSED
            except BaseException as exc:  # carried across the C boundary
                raised.append(exc)
                return self._ISSUE_FAILED

        e_arr, e_n = _ints(experts)
        r_arr, r_n = _ints(resident)
        rc = capi.load().shrike_prefetch_ring_begin(self._h, layer, e_arr, e_n, r_arr, r_n, 1 if deferred else 0,
                                                    capi.PREFETCH_ISSUE(trampoline), None)
        if rc:
            for item in raised:
                if isinstance(item, BaseException):
                    raise item
            raise ShrikeError(f"prefetch begin failed (code {rc})")

    def ready_cells(self, layer: int, experts, join_nanos: int = 0) -> dict:
        e_arr, e_n = _ints(experts)
        out_e, out_c = (C.c_int * max(1, e_n))(), (C.c_int * max(1, e_n))()
        n = capi.load().shrike_prefetch_ring_ready_cells(self._h, layer, e_arr, e_n, join_nanos, out_e, out_c)
        return {out_e[i]: out_c[i] for i in range(n)}

    def consume(self, layer: int, experts, freed_cells: dict) -> None:
        e_arr, e_n = _ints(experts)
        f_e, f_n = _ints(freed_cells.keys())
        f_c, _ = _ints(freed_cells.values())
        capi.load().shrike_prefetch_ring_consume(self._h, layer, e_arr, e_n, f_e, f_c, f_n)

    def claim_demand(self, layer: int, experts) -> dict:
        e_arr, e_n = _ints(experts)
        out_e, out_c = (C.c_int * max(1, e_n))(), (C.c_int * max(1, e_n))()
        n = capi.load().shrike_prefetch_ring_claim_demand(self._h, layer, e_arr, e_n, out_e, out_c)
        return {out_e[i]: out_c[i] for i in range(n)}

    def attach_demand(self, layer: int, experts, operation: ExpertLoadOperation) -> None:
        e_arr, e_n = _ints(experts)
        capi.load().shrike_prefetch_ring_attach_demand(self._h, layer, e_arr, e_n, operation._h)

    def completion_nanos(self, layer: int, experts) -> dict:
        e_arr, e_n = _ints(experts)
        out_e, out_t = (C.c_int * max(1, e_n))(), (C.c_uint64 * max(1, e_n))()
        n = capi.load().shrike_prefetch_ring_completion_nanos(self._h, layer, e_arr, e_n, out_e, out_t)
        return {out_e[i]: int(out_t[i]) for i in range(n)}

    def unlease(self, layer: int, experts) -> None:
        e_arr, e_n = _ints(experts)
        capi.load().shrike_prefetch_ring_unlease(self._h, layer, e_arr, e_n)

    def note_demand_submission(self) -> None:
        capi.load().shrike_prefetch_ring_note_demand_submission(self._h)

    def note_hook_failure(self) -> bool:
        return bool(capi.load().shrike_prefetch_ring_note_hook_failure(self._h))

    @property
    def statistics(self) -> dict:
        st = capi.PrefetchStatistics()
        capi.load().shrike_prefetch_ring_statistics(self._h, C.byref(st))
        return {name: int(getattr(st, name)) for name, _ in capi.PrefetchStatistics._fields_}

    @property
    def in_flight_count(self) -> int:
        return capi.load().shrike_prefetch_ring_in_flight_count(self._h)

    @property
    def leased_count(self) -> int:
        return capi.load().shrike_prefetch_ring_leased_count(self._h)
