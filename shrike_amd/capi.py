"""ctypes binding of libshrikehip.so (include/shrike_hip.h).

The library is the product; this module only declares its entry points. There is
no fallback: if the shared object is missing or a call fails, an exception says so.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# SHRIKE_HIP_LIBRARY names another build of the same library (kernel experiments)
LIB_PATH = os.environ.get("SHRIKE_HIP_LIBRARY") or os.path.join(_HERE, "libshrikehip.so")

MAX_TOP_K = 8
POOL_MAX_CHUNKS = 8
SENTINEL = 0xFFFFFFFF
POOL_PAGE = 16384
META_BF16, META_F16 = 0, 1
ACT_GELU_TANH, ACT_SILU, ACT_CLAMPED_SWIGLU = 0, 1, 2
EMPTY, LOADING, RESIDENT = 0, 1, 2


class ShrikeError(RuntimeError):
    pass


class ExpertOffsets(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in (
        "gate_w_off", "gate_s_off", "gate_b_off", "up_w_off", "up_s_off", "up_b_off",
        "down_w_off", "down_s_off", "down_b_off", "gate_ab_off", "up_ab_off", "down_ab_off")]


class PoolBases(C.Structure):
    _fields_ = [("base", C.c_void_p * POOL_MAX_CHUNKS), ("cells_per_chunk", C.c_uint32)]


class Projection(C.Structure):
    _fields_ = [("weights", C.c_void_p), ("scales", C.c_void_p), ("biases", C.c_void_p)]


class RouterOperands(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("weights", "scales", "biases", "effective_scale", "logit_bias",
                                          "out_indices", "out_weights")]


class MoEDesc(C.Structure):
    _fields_ = [("d", C.c_uint32), ("f", C.c_uint32), ("num_experts", C.c_uint32),
                ("top_k", C.c_uint32), ("routed_weight_bits", C.c_uint32),
                ("router_weight_bits", C.c_uint32), ("meta_dtype", C.c_uint32),
                ("activation", C.c_uint32), ("expert_additive_biases", C.c_uint32),
                ("sigmoid_router_scores", C.c_uint32), ("routed_scaling_factor", C.c_float),
                ("event_gated_io", C.c_uint32)]


class DecodeLayerArgs(C.Structure):
    _fields_ = [
        ("router_weights", C.c_void_p), ("router_scales", C.c_void_p), ("router_biases", C.c_void_p),
        ("effective_scale", C.c_void_p), ("per_expert_scale", C.c_void_p), ("logit_bias", C.c_void_p),
        ("pool", C.POINTER(PoolBases)), ("pool_slot_stride", C.c_uint64), ("residency", C.c_void_p),
        ("offsets", ExpertOffsets),
        ("shared_gate", Projection), ("shared_up", Projection), ("shared_down", Projection),
        ("shared_bits", C.c_uint32), ("shared_f", C.c_uint32), ("shared_scalar_gate", C.c_void_p),
        ("x", C.c_void_p), ("hidden", C.c_void_p), ("y", C.c_void_p),
        ("out_indices", C.c_void_p), ("out_weights", C.c_void_p),
        ("resolved_slots", C.c_void_p), ("hit_count", C.c_void_p), ("hit_positions", C.c_void_p),
        ("miss_count", C.c_void_p), ("miss_positions", C.c_void_p), ("miss_experts", C.c_void_p),
        ("acts", C.c_void_p), ("shared_scratch", C.c_void_p), ("h1", C.c_void_p),
        ("norm_delta", C.c_void_p), ("norm_weight", C.c_void_p), ("norm_eps", C.c_float)]


# name -> (restype, argtypes); every symbol include/shrike_hip.h declares
_VP, _U32, _U64, _I32, _I64 = C.c_void_p, C.c_uint32, C.c_uint64, C.c_int32, C.c_int64
class RowTile(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("cell", "pair_start", "rows", "expert")]


class HipGroupedRoutes(C.Structure):
    _fields_ = [("sorted_pairs", C.c_void_p), ("per_expert_offsets", C.c_void_p), ("per_expert_counts", C.c_void_p),
                ("row_tiles", C.c_void_p), ("row_tile_count", C.c_void_p)]


# ---- include/shrike_host.h ----------------------------------------------------------

class TokenExpertPair(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("token", "expert", "rank", "weight_bits_and_reserved")]


class MoEGroup(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("expert", "pair_start", "pair_count")]


class MoETile(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("group_start", "group_count", "pair_start", "pair_count")]


class GroupedRoutes(C.Structure):
    _fields_ = [("sorted_pairs", C.POINTER(TokenExpertPair)), ("per_expert_offsets", C.POINTER(C.c_uint32)),
                ("per_expert_counts", C.POINTER(C.c_uint32)), ("groups", C.POINTER(MoEGroup)),
                ("tiles", C.POINTER(MoETile)), ("group_count", C.c_uint32), ("tile_count", C.c_uint32),
                ("max_pairs_per_expert", C.c_uint32), ("max_pairs_per_tile", C.c_uint32),
                ("max_live_experts_per_tile", C.c_uint32), ("error_value", C.c_int64 * 2)]


class ExpertPairRange(C.Structure):
    _fields_ = [("expert", C.c_uint32), ("pair_start", C.c_int64), ("pair_count", C.c_int64)]


class RoutedExpertBlock(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("slot", "pair_start", "rows", "staging_row", "row_tile_start")]


class RoutedExpertWave(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("block_start", "block_count", "padded_rows", "tail_rows")]


class ExpertCachePlan(C.Structure):
    _fields_ = [("expert_count", C.c_uint32), ("layer", C.c_int32), ("experts", C.POINTER(C.c_int32)),
                ("assigned_slots", C.POINTER(C.c_int32)), ("assigned_generations", C.POINTER(C.c_uint64)),
                ("misses", C.POINTER(C.c_uint32)), ("miss_count", C.c_uint32), ("hits", C.c_uint32),
                ("assigned_cells", C.POINTER(C.c_uint32)), ("adopted", C.POINTER(C.c_uint32)),
                ("adopted_count", C.c_uint32), ("freed_count", C.c_uint32),
                ("freed_experts", C.POINTER(C.c_int32)), ("freed_cells", C.POINTER(C.c_uint32))]


class StreamingStatistics(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in (
        "plans", "requested_experts", "hits", "misses", "bytes_read", "read_operations", "evictions",
        "reloads", "load_batches", "total_load_nanos", "fetch_nanos", "maximum_load_nanos")] + [
        ("latency_histogram", C.c_uint64 * 17)] + [(n, C.c_uint32) for n in (
            "resident_slots", "loading_slots", "pinned_slots", "peak_loading_slots")]


class ExpertBatchSlot(C.Structure):
    _fields_ = [("active", C.c_int), ("sequence", C.c_uint64), ("next_index", C.c_size_t), ("count", C.c_size_t)]


class ExpertBatchCancelState(C.Structure):
    _fields_ = [("count", C.c_size_t), ("next_index", C.c_size_t), ("outstanding", C.c_size_t),
                ("first_errno", C.c_int)]


class PackedExpert(C.Structure):
    _fields_ = [("expert", C.c_int32), ("physical_rank", C.c_int32), ("offset", C.c_uint64), ("size", C.c_uint64),
                ("tensor_count", C.c_uint32)]


class PackedTensor(C.Structure):
    _fields_ = [("offset", C.c_uint64), ("size", C.c_uint64), ("dtype", C.c_char * 8), ("shape", C.c_uint32 * 4),
                ("rank", C.c_uint32), ("bits", C.c_int32)]


class TileSchedulerConfig(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("max_pending_depth", "tile_experts", "tiles_per_command_buffer", "fetch_lookahead")]


class TileBatchAction(C.Structure):
    _fields_ = [("commit_before_append", C.c_int32), ("commit_after_append", C.c_int32)]


class TileDriver(C.Structure):
    _fields_ = [("context", C.c_void_p),
                ("open_batch_tiles", C.CFUNCTYPE(C.c_int, C.c_void_p)),
                ("open_batch_slot_count", C.CFUNCTYPE(C.c_size_t, C.c_void_p)),
                ("pending_depth", C.CFUNCTYPE(C.c_int, C.c_void_p)),
                ("pending_assigned_slot_count", C.CFUNCTYPE(C.c_size_t, C.c_void_p)),
                ("plan", C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_int))),
                ("begin", C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int)),
                ("abandon_plan", C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int)),
                ("encode", C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int)),
                ("commit_open_batch", C.CFUNCTYPE(None, C.c_void_p)),
                ("drain_oldest_batch", C.CFUNCTYPE(C.c_int, C.c_void_p)),
                ("abandon_begun_fetches", C.CFUNCTYPE(None, C.c_void_p))]


class PrefetchStatistics(C.Structure):
    _fields_ = [(name, C.c_uint64) for name in ("issued", "adopted", "reclaimed", "deferred", "overlapped", "late", "joined",
                                                "refused", "failed", "hook_failures", "begin_nanos", "leased_peak")]


PREFETCH_DROP = C.CFUNCTYPE(None, C.c_void_p, C.c_int, C.c_int, C.c_int)
PREFETCH_ISSUE = C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(C.c_int), C.POINTER(C.c_int), C.c_size_t, C.POINTER(C.c_void_p))


class RouterReadback(C.Structure):
    _fields_ = [("hit_count", C.c_uint32), ("miss_count", C.c_uint32), ("expert_ids", C.c_uint32 * 8),
                ("weight_bits", C.c_uint16 * 8), ("hit_positions", C.c_uint32 * 8), ("miss_positions", C.c_uint32 * 8),
                ("predicted_ids", C.c_uint32 * 8)]


class IOCompletionToken(C.Structure):
    _fields_ = [("value", C.c_uint64), ("status_index", C.c_uint32), ("status", C.POINTER(C.c_uint32))]


IO_WORK = C.CFUNCTYPE(None, C.c_void_p)

SIGNATURES = {
    "shrike_hip_last_error": (C.c_char_p, []),
    "shrike_hip_moe_decode_layer_batch": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(DecodeLayerArgs), C.c_uint32, C.c_uint32]),
    "shrike_int4_affine_gemv": (None, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p]),
    "shrike_cpu_expert_ffn_scratch_floats": (C.c_size_t, [C.c_uint32, C.c_uint32]),
    "shrike_cpu_expert_ffn_accumulate": (C.c_int, [C.c_void_p, C.POINTER(ExpertOffsets), C.c_void_p, C.c_uint32, C.c_uint32,
                                                   C.c_float, C.c_void_p, C.c_void_p]),
    "shrike_load_acquire_u32": (C.c_uint32, [C.c_void_p]),
    "shrike_store_release_u64": (None, [C.c_void_p, C.c_uint64]),
    "shrike_router_readback_word_count": (C.c_uint32, [C.c_uint32]),
    "shrike_router_readback_word": (C.c_uint32, [C.c_uint32, C.c_uint32]),
    "shrike_router_readback_next_tag": (C.c_uint32, [C.c_uint32]),
    "shrike_router_readback_is_complete": (C.c_int, [C.c_void_p, C.c_uint32, C.c_uint32]),
    "shrike_router_readback_decode": (C.c_int, [C.c_void_p, C.c_uint32, C.c_uint32, C.POINTER(RouterReadback)]),
    "shrike_router_readback_poll": (C.c_int, [C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint64, C.POINTER(RouterReadback)]),
    "shrike_io_scheduler_create": (C.c_void_p, [C.c_int, C.POINTER(C.c_int)]),
    "shrike_io_scheduler_submit": (C.c_int, [C.c_void_p, C.c_int, IO_WORK, C.c_void_p]),
    "shrike_io_scheduler_close": (None, [C.c_void_p]),
    "shrike_io_scheduler_destroy": (None, [C.c_void_p]),
    "shrike_io_scheduler_workers": (C.c_int, [C.c_void_p]),
    "shrike_io_timeline_create": (C.c_void_p, [C.c_void_p, C.c_uint32, C.POINTER(C.c_int)]),
    "shrike_io_timeline_destroy": (None, [C.c_void_p]),
    "shrike_io_timeline_reserve": (C.c_int, [C.c_void_p, C.POINTER(IOCompletionToken)]),
    "shrike_io_timeline_publish": (C.c_uint64, [C.c_void_p, C.POINTER(IOCompletionToken), C.c_int]),
    "shrike_io_timeline_published": (C.c_uint64, [C.c_void_p]),
    "shrike_tile_scheduler_config_make": (None, [C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(TileSchedulerConfig)]),
    "shrike_tile_scheduler_fits_slot_budget": (C.c_int, [C.POINTER(TileSchedulerConfig), C.c_int, C.c_int]),
    "shrike_tile_scheduler_fitting": (C.c_int, [C.POINTER(TileSchedulerConfig), C.c_int, C.c_int, C.POINTER(TileSchedulerConfig)]),
    "shrike_tile_scheduler_decide": (C.c_int, [C.POINTER(TileSchedulerConfig), C.c_int, C.c_int, C.c_size_t, C.c_int]),
    "shrike_tile_scheduler_plans_lookahead": (C.c_int, [C.POINTER(TileSchedulerConfig), C.c_int, C.c_int]),
    "shrike_tile_scheduler_should_begin_lookahead": (C.c_int, [C.POINTER(TileSchedulerConfig), C.c_int, C.c_int, C.c_int]),
    "shrike_tile_scheduler_batch_action": (None, [C.POINTER(TileSchedulerConfig), C.c_int, C.c_size_t, C.c_int, C.c_int,
                                                  C.POINTER(TileBatchAction)]),
    "shrike_tile_sequencer_run": (C.c_int, [C.POINTER(TileSchedulerConfig), C.c_int, C.POINTER(TileDriver)]),
    "shrike_chunk_protection_init": (None, [C.POINTER(C.c_int32), C.c_size_t, C.POINTER(C.c_uint8), C.c_size_t]),
    "shrike_chunk_protection_planning": (None, [C.POINTER(C.c_int32), C.c_size_t, C.POINTER(C.c_uint8), C.c_size_t]),
    "shrike_tile_lifetime_create": (_VP, []),
    "shrike_tile_lifetime_destroy": (None, [_VP]),
    "shrike_tile_lifetime_begin": (C.c_int, [_VP, C.c_int, C.POINTER(C.c_int32), C.c_size_t, C.POINTER(C.c_int)]),
    "shrike_tile_lifetime_complete": (C.c_int, [_VP, C.c_int]),
    "shrike_monotonic_nanos": (C.c_uint64, []),
    "shrike_load_operation_create": (_VP, []),
    "shrike_load_operation_retain": (None, [_VP]),
    "shrike_load_operation_release": (None, [_VP]),
    "shrike_load_operation_state": (C.c_int, [_VP]),
    "shrike_load_operation_mark_in_flight": (C.c_int, [_VP]),
    "shrike_load_operation_finish": (C.c_int, [_VP, C.c_int]),
    "shrike_load_operation_wait": (C.c_int, [_VP]),
    "shrike_load_operation_wait_until": (C.c_int, [_VP, C.c_uint64]),
    "shrike_load_operation_submitted_nanos": (C.c_uint64, [_VP]),
    "shrike_load_operation_started_nanos": (C.c_uint64, [_VP]),
    "shrike_load_operation_completed_nanos": (C.c_uint64, [_VP]),
    "shrike_prefetch_ring_create": (_VP, [C.POINTER(C.c_int), C.c_size_t, PREFETCH_DROP, C.c_void_p, C.POINTER(C.c_int)]),
    "shrike_prefetch_ring_destroy": (None, [_VP]),
    "shrike_prefetch_ring_begin": (C.c_int, [_VP, C.c_int, C.POINTER(C.c_int), C.c_size_t, C.POINTER(C.c_int), C.c_size_t, C.c_int,
                                             PREFETCH_ISSUE, C.c_void_p]),
    "shrike_prefetch_ring_ready_cells": (C.c_size_t, [_VP, C.c_int, C.POINTER(C.c_int), C.c_size_t, C.c_uint64, C.POINTER(C.c_int),
                                                      C.POINTER(C.c_int)]),
    "shrike_prefetch_ring_consume": (None, [_VP, C.c_int, C.POINTER(C.c_int), C.c_size_t, C.POINTER(C.c_int), C.POINTER(C.c_int),
                                            C.c_size_t]),
    "shrike_prefetch_ring_claim_demand": (C.c_size_t, [_VP, C.c_int, C.POINTER(C.c_int), C.c_size_t, C.POINTER(C.c_int),
                                                       C.POINTER(C.c_int)]),
    "shrike_prefetch_ring_attach_demand": (None, [_VP, C.c_int, C.POINTER(C.c_int), C.c_size_t, _VP]),
    "shrike_prefetch_ring_completion_nanos": (C.c_size_t, [_VP, C.c_int, C.POINTER(C.c_int), C.c_size_t, C.POINTER(C.c_int),
                                                           C.POINTER(C.c_uint64)]),
    "shrike_prefetch_ring_unlease": (None, [_VP, C.c_int, C.POINTER(C.c_int), C.c_size_t]),
    "shrike_prefetch_ring_note_demand_submission": (None, [_VP]),
    "shrike_prefetch_ring_note_hook_failure": (C.c_int, [_VP]),
    "shrike_prefetch_ring_statistics": (None, [_VP, C.POINTER(PrefetchStatistics)]),
    "shrike_prefetch_ring_in_flight_count": (C.c_int, [_VP]),
    "shrike_prefetch_ring_leased_count": (C.c_int, [_VP]),
    "shrike_host_last_error": (C.c_char_p, []),
    "shrike_expert_reader_create": (_VP, [C.c_char_p, C.c_size_t, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_int)]),
    "shrike_expert_reader_destroy": (None, [_VP]),
    "shrike_expert_reader_fetch": (C.c_int, [_VP, C.POINTER(C.c_uint32), C.POINTER(C.c_void_p), C.c_size_t]),
    "shrike_expert_reader_fetch_offsets": (C.c_int, [_VP, C.POINTER(C.c_uint64), C.POINTER(C.c_void_p), C.c_size_t]),
    "shrike_expert_reader_threads": (C.c_int, [_VP]),
    "shrike_expert_reader_batch_depth": (C.c_int, [_VP]),
    "shrike_expert_reader_claim_slot": (C.c_int, [C.POINTER(ExpertBatchSlot), C.c_int]),
    "shrike_expert_reader_free_slot": (C.c_int, [C.POINTER(ExpertBatchSlot), C.c_int]),
    "shrike_expert_reader_cancel_slot": (None, [C.POINTER(ExpertBatchCancelState)]),
    "shrike_packed_layout_decode": (_VP, [C.c_char_p, C.c_size_t, C.POINTER(C.c_int)]),
    "shrike_packed_layout_load": (_VP, [C.c_char_p, C.c_uint64, C.POINTER(C.c_int)]),
    "shrike_packed_layout_destroy": (None, [_VP]),
    "shrike_packed_layout_expert_stride": (C.c_uint64, [_VP]),
    "shrike_packed_layout_num_layers": (C.c_int, [_VP]),
    "shrike_packed_layout_experts_per_layer": (C.c_int, [_VP]),
    "shrike_packed_layout_layer": (C.c_int, [_VP, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_char_p), C.POINTER(C.c_int)]),
    "shrike_packed_layout_expert": (C.c_int, [_VP, C.c_int, C.c_int, C.POINTER(PackedExpert)]),
    "shrike_packed_layout_tensor": (C.c_int, [_VP, C.c_int, C.c_int, C.c_char_p, C.POINTER(PackedTensor)]),
    "shrike_packed_layout_expert_offsets": (C.c_int, [_VP, C.c_int, C.c_int, C.POINTER(ExpertOffsets)]),
    "shrike_packed_layout_cross_validate": (C.c_int, [_VP, C.c_int, C.c_int, C.c_uint64, C.POINTER(C.c_char_p),
                                                      C.POINTER(C.c_uint64), C.c_size_t]),
    "shrike_hip_init": (C.c_int, [C.c_int]),
    "shrike_expert_offsets_make": (_U64, [_U32, _U32, _U32, C.c_int, C.POINTER(ExpertOffsets)]),
    "shrike_parse_budget_bytes": (_I64, [C.c_char_p]),
    "shrike_expert_cache_slots": (_I32, [_U64, _I32, _I64]),
    "shrike_hip_pool_create": (_VP, [_U32, _U64, _U32, _U64, C.POINTER(C.c_int)]),
    "shrike_hip_pool_create_layer_view": (_VP, [_VP, _U32, C.POINTER(C.c_int)]),
    "shrike_hip_pool_destroy": (None, [_VP]),
    "shrike_hip_pool_fetch_experts": (C.c_int, [_VP, _VP, _VP, C.POINTER(C.c_uint64), C.POINTER(C.c_uint32), _U32, _U64,
                                                _VP, _U64]),
    "shrike_hip_pool_slot_stride": (_U64, [_VP]),
    "shrike_hip_pool_cell_count": (_U32, [_VP]),
    "shrike_hip_pool_cell_ptr": (_VP, [_VP, _U32]),
    "shrike_hip_pool_bases": (C.POINTER(PoolBases), [_VP]),
    "shrike_hip_pool_residency_table": (_VP, [_VP]),
    "shrike_hip_pool_upload_async": (C.c_int, [_VP, _U32, _VP, _U64, _VP]),
    "shrike_hip_pool_table_publish": (C.c_int, [_VP, _U32, _U32, _U32, _VP]),
    "shrike_hip_pool_table_entry": (_U64, [_VP, _U32]),
    "shrike_hip_moe_create": (_VP, [C.POINTER(MoEDesc), C.POINTER(C.c_int)]),
    "shrike_hip_moe_destroy": (None, [_VP]),
    "shrike_hip_moe_router": (C.c_int, [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP,
                                        _U32, _U32, _U32]),
    "shrike_hip_moe_router_logits": (_VP, [_VP]),
    "shrike_hip_moe_router_pair": (C.c_int, [_VP, _VP, C.POINTER(RouterOperands), C.POINTER(RouterOperands), _VP, _VP,
                                             _U32, _U32, _U32, _VP]),
    "shrike_hip_moe_router_pair_logits": (_VP, [_VP]),
    "shrike_hip_shared_scalar_gate_rows": (C.c_int, [_VP, C.POINTER(Projection), _U32, _VP, _U32, _VP, _U32, _U32]),
    "shrike_hip_sigmoid_scalar_mul_rows": (C.c_int, [_VP, _VP, _VP, _U32, _U32]),
    "shrike_hip_moe_classify": (C.c_int, [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _U32, _U32,
                                          C.POINTER(_U32), _VP, _VP, _U32, _VP, _VP]),
    "shrike_hip_moe_phase1_pool": (C.c_int, [_VP, _VP, C.POINTER(PoolBases), _U64, _VP,
                                             C.POINTER(ExpertOffsets), _VP, _VP, _U32, _U32, _U32,
                                             _VP, _VP]),
    "shrike_hip_moe_phase2_pool": (C.c_int, [_VP, _VP, C.POINTER(PoolBases), _U64, _VP, _VP,
                                             C.POINTER(ExpertOffsets), _VP, _VP, _VP, _VP, _VP,
                                             _U32, _U32, _U32, _VP, _VP]),
    "shrike_hip_moe_phase1_blobs": (C.c_int, [_VP, _VP, _VP, C.POINTER(ExpertOffsets), _VP, _VP, _U32, _U32, _U32, _VP, _U32, _VP]),
    "shrike_hip_moe_phase2_blobs": (C.c_int, [_VP, _VP, _VP, C.POINTER(ExpertOffsets), _VP, _VP, _VP, _VP, _VP, _U32, _U32, _U32, _VP]),
    "shrike_hip_shared_expert": (C.c_int, [_VP, _VP, C.POINTER(Projection), C.POINTER(Projection),
                                           C.POINTER(Projection), _U32, _VP, _VP, _VP, _VP, _U32, _U32]),
    "shrike_hip_moe_decode_layer": (C.c_int, [_VP, _VP, C.POINTER(DecodeLayerArgs)]),
    "shrike_hip_moe_decode_layer_launches": (C.c_int, [_VP, _VP, C.POINTER(DecodeLayerArgs), _U32]),
    "shrike_hip_moe_decode_layer_noalloc": (C.c_int, [C.POINTER(MoEDesc), _VP, C.POINTER(DecodeLayerArgs)]),
    "shrike_hip_residual_add_rmsnorm_bf16w": (C.c_int, [_VP, _VP, _VP, _VP, _VP, _U32, C.c_float, _U32]),
    "shrike_hip_malloc": (_VP, [_U64]),
    "shrike_hip_free": (C.c_int, [_VP]),
    "shrike_hip_host_alloc": (_VP, [_U64]),
    "shrike_hip_host_free": (C.c_int, [_VP]),
    "shrike_hip_memcpy_h2d": (C.c_int, [_VP, _VP, _U64]),
    "shrike_hip_memcpy_d2h": (C.c_int, [_VP, _VP, _U64]),
    "shrike_hip_memcpy_d2d": (C.c_int, [_VP, _VP, _U64]),
    "shrike_hip_memcpy_h2d_async": (C.c_int, [_VP, _VP, _U64, _VP]),
    "shrike_hip_memset": (C.c_int, [_VP, C.c_int, _U64]),
    "shrike_hip_device_synchronize": (C.c_int, []),
    "shrike_hip_mem_info": (C.c_int, [C.POINTER(_U64), C.POINTER(_U64)]),
    "shrike_hip_stream_create": (_VP, []),
    "shrike_hip_stream_destroy": (C.c_int, [_VP]),
    "shrike_hip_stream_synchronize": (C.c_int, [_VP]),
    "shrike_hip_event_create": (_VP, []),
    "shrike_hip_event_destroy": (C.c_int, [_VP]),
    "shrike_hip_event_record": (C.c_int, [_VP, _VP]),
    "shrike_hip_event_synchronize": (C.c_int, [_VP]),
    "shrike_hip_stream_wait_event": (C.c_int, [_VP, _VP]),
    "shrike_hip_event_elapsed_ms": (C.c_int, [_VP, _VP, C.POINTER(C.c_float)]),
    "shrike_hip_graph_begin_capture": (C.c_int, [_VP]),
    "shrike_hip_graph_end_capture": (_VP, [_VP]),
    "shrike_hip_graph_launch": (C.c_int, [_VP, _VP]),
    "shrike_hip_graph_destroy": (C.c_int, [_VP]),
    "shrike_hip_pool_execute_plan": (C.c_int, [_VP, _VP, C.POINTER(ExpertCachePlan), _VP, _U64, _U64, _VP, _U64]),
    "shrike_hip_moe_resolve_batch": (C.c_int, [_VP, _VP, _VP, _VP, _U32, _U32, _VP]),
    "shrike_hip_moe_phase1_batch": (C.c_int, [_VP, _VP, C.POINTER(PoolBases), _U64, _VP, C.POINTER(ExpertOffsets), _VP, _U32, _VP,
                                              _U32, _U32, _U32, _U32]),
    "shrike_hip_moe_phase2_batch": (C.c_int, [_VP, _VP, C.POINTER(PoolBases), _U64, _VP, C.POINTER(ExpertOffsets), _VP, _VP, _VP, _VP,
                                              _VP, _U32, _U32, _U32, _U32]),
    # prefill operators
    "shrike_hip_prefill_router": (C.c_int, [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP,
                                            _U32, _U32, _U32, _U32, _U32]),
    "shrike_hip_prefill_router_with_group_sums": (C.c_int, [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP,
                                                            _U32, _U32, _U32, _U32, _U32, _VP]),
    "shrike_hip_prefill_router_workspace_bytes": (C.c_size_t, [_U32, _U32, _U32]),
    "shrike_hip_group_max_row_tiles": (_U32, [_U64, _U32]),
    "shrike_hip_group_pairs": (C.c_int, [_VP, _VP, _VP, _U32, _U32, _U32, _VP, _VP, C.POINTER(HipGroupedRoutes)]),
    "shrike_hip_prefill_ffn_workspace_bytes": (C.c_size_t, [_U32, _U32, _U32, _U32]),
    "shrike_hip_prefill_grouped_ffn": (C.c_int, [_VP, _VP, C.POINTER(PoolBases), _U64, C.POINTER(ExpertOffsets),
                                                 C.POINTER(HipGroupedRoutes), _U32, _VP, _U32, _VP, _VP, C.c_size_t,
                                                 _U32, _U32, _U32, _U32]),
    "shrike_hip_prefill_grouped_ffn_presummed": (C.c_int, [_VP, _VP, C.POINTER(PoolBases), _U64, C.POINTER(ExpertOffsets),
                                                           C.POINTER(HipGroupedRoutes), _U32, _VP, _U32, _VP, _VP, C.c_size_t,
                                                           _U32, _U32, _U32, _U32]),
    "shrike_hip_prefill_streamed_batched": (C.c_int, [_VP, _VP, C.POINTER(PoolBases), _U64, C.POINTER(ExpertOffsets),
                                                      C.POINTER(HipGroupedRoutes), _U32, _VP, _U32, _U32, _U32, _VP, _U32,
                                                      _VP, _VP, C.c_size_t, _U32, _U32, _U32, _U32, C.POINTER(C.c_uint32)]),
    "shrike_hip_prefill_shared_expert_workspace_bytes": (C.c_size_t, [_U32, _U32, _U32]),
    "shrike_hip_prefill_shared_expert": (C.c_int, [_VP, _VP, C.POINTER(Projection), C.POINTER(Projection), C.POINTER(Projection),
                                                   _U32, _VP, _U32, _VP, _VP, _VP, C.c_size_t, _U32, _U32, _U32]),
    "shrike_hip_prefill_reduce": (C.c_int, [_VP, _VP, _VP, _VP, _U32, _U32, _U32]),
    "shrike_hip_residual_add_f16": (C.c_int, [_VP, _VP, _VP, _U64]),
    # include/shrike_host.h
    "shrike_make_token_expert_pairs": (C.c_int, [_VP, _VP, _U32, _U32, C.POINTER(TokenExpertPair)]),
    "shrike_group_pairs": (C.c_int, [C.POINTER(TokenExpertPair), C.c_size_t, _I64, _I64, _I64, _I64, _VP,
                                     C.c_size_t, C.POINTER(GroupedRoutes)]),
    "shrike_sweep_order_resident_first_balanced": (C.c_int, [_VP, _VP, _VP, C.c_size_t, _VP, C.c_size_t, _I64, _I64,
                                                             _VP, C.POINTER(C.c_size_t)]),
    "shrike_expert_sort_keys": (None, [_VP, C.c_size_t, C.c_size_t, _VP]),
    "shrike_plan_expert_waves": (C.c_int, [C.POINTER(ExpertPairRange), C.c_size_t, _VP, C.c_size_t, _I64, _I64, _I64,
                                           C.POINTER(RoutedExpertBlock), C.c_size_t, C.POINTER(C.c_size_t),
                                           C.POINTER(RoutedExpertWave), C.c_size_t, C.POINTER(C.c_size_t)]),
    "shrike_row_tile_table": (C.c_int, [C.POINTER(RoutedExpertBlock), C.c_size_t, _U32, _U32, _VP]),
    "shrike_row_tile_tables": (C.c_int, [C.POINTER(RoutedExpertBlock), C.c_size_t, _U32, _U32, _VP, _VP, _VP]),
    "shrike_slot_cache_create": (_VP, [_U32, _U32, _U32, C.c_int, C.c_double, C.POINTER(C.c_int)]),
    "shrike_slot_cache_destroy": (None, [_VP]),
    "shrike_cell_arena_create": (_VP, [_U32, C.POINTER(C.c_int)]),
    "shrike_cell_arena_destroy": (None, [_VP]),
    "shrike_cell_arena_cell_count": (_U32, [_VP]),
    "shrike_cell_arena_generation": (_U64, [_VP, _U32]),
    "shrike_slot_cache_create_in_arena": (_VP, [_VP, _U32, _U32, _U32, C.c_int, C.c_double, C.POINTER(C.c_int)]),
    "shrike_slot_cache_plan_with_landings": (C.c_int, [_VP, _VP, _U32, _I32, _VP, _U32, _VP, _U32, _VP, _U32, _VP, _U32,
                                                       _I64, C.POINTER(ExpertCachePlan)]),
    "shrike_slot_cache_slot_cell": (_I64, [_VP, _U32]),
    "shrike_slot_cache_owns_cell": (C.c_int, [_VP, _U32]),
    "shrike_slot_cache_claim_landing": (C.c_int, [_VP, _I32, _I64]),
    "shrike_slot_cache_complete_landing": (C.c_int, [_VP, _I32, _I64]),
    "shrike_slot_cache_fail_landing": (None, [_VP, _I32, _I64]),
    "shrike_slot_cache_drop_landing": (None, [_VP, _I32, _I64]),
    "shrike_slot_cache_claim_prefetch": (C.c_int, [_VP, _VP, _VP, _U32, C.POINTER(C.c_uint32)]),
    "shrike_slot_cache_reserve_overflow_slot": (_I64, [_VP, _I32, _VP, _U32]),
    "shrike_slot_cache_mark_overflow_resident": (None, [_VP, _I32, _I64]),
    "shrike_slot_cache_abandon_overflow_slot": (None, [_VP, _I32, _I64]),
    "shrike_slot_cache_finish_agreed_reads": (C.c_int, [_VP, _VP, _VP, _U32, C.c_int, _U64, _U64]),
    "shrike_slot_cache_plan": (C.c_int, [_VP, _VP, _U32, _I32, _VP, _U32, _VP, _U32, _I64, C.POINTER(ExpertCachePlan)]),
    "shrike_slot_cache_complete": (C.c_int, [_VP, C.POINTER(ExpertCachePlan), _U64, _U64]),
    "shrike_slot_cache_abandon": (None, [_VP, C.POINTER(ExpertCachePlan)]),
    "shrike_slot_cache_pin": (C.c_int, [_VP, C.POINTER(ExpertCachePlan)]),
    "shrike_slot_cache_unpin": (None, [_VP, _VP, _VP, _U32]),
    "shrike_slot_cache_statistics": (None, [_VP, _U64, C.POINTER(StreamingStatistics)]),
    "shrike_slot_cache_resident_experts": (C.c_size_t, [_VP, _VP, C.c_size_t]),
    "shrike_slot_cache_entry": (_U64, [_VP, _U32]),
    "shrike_slot_cache_drain_publications": (C.c_size_t, [_VP, _VP, _VP, C.c_size_t]),
}

_lib = None


def load() -> C.CDLL:
    """Load the built library; raise if it has not been built (no fallback exists)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ShrikeError(
                f"{LIB_PATH} is missing: build it first (python -c 'import __graft_entry__ as g; g.build()')")
        lib = C.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
            fn.restype, fn.argtypes = restype, argtypes
        _lib = lib
    return _lib


def last_error() -> str:
    return load().shrike_hip_last_error().decode("utf-8", "replace")


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise ShrikeError(f"{what} failed with {rc} ({os.strerror(rc)}): {last_error()}")
