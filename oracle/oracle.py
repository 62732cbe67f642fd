"""TEST INFRASTRUCTURE — NOT PRODUCT CODE.

ctypes face of liboracle.so (oracle/shrike_oracle.c), the scalar CPU restatement
of Shrike's routed-expert arithmetic. Only tests/, __graft_entry__.smoke() and
bench.py's cpu_baseline leg may import this module, and only as the checker.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
META_BF16, META_F16 = 0, 1
ACT_GELU_TANH, ACT_SILU, ACT_CLAMPED_SWIGLU = 0, 1, 2
ROUTER_F16, ROUTER_AFFINE8, ROUTER_AFFINE4 = 0, 8, 4


class Offsets(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in (
        "gate_w", "gate_s", "gate_b", "up_w", "up_s", "up_b",
        "down_w", "down_s", "down_b", "gate_ab", "up_ab", "down_ab")]

    def as_tuple(self):
        return tuple(getattr(self, n) for n, _ in self._fields_)


class Proj(C.Structure):
    _fields_ = [("w", C.c_void_p), ("s", C.c_void_p), ("b", C.c_void_p)]


def build(force: bool = False) -> str:
    """Compile liboracle.so (and oracle/_ref when the reference checkout exists)."""
    path = os.path.join(_HERE, "liboracle.so")
    if force or not os.path.exists(path):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s", "all"], check=True,
                       stdout=subprocess.DEVNULL)
    return path


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
        L = _lib
        L.orc_f32_to_bf16.restype = C.c_uint16
        L.orc_f32_to_bf16.argtypes = [C.c_float]
        L.orc_bf16_to_f32.restype = C.c_float
        L.orc_bf16_to_f32.argtypes = [C.c_uint16]
        L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [C.c_float]
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_glu.restype = C.c_float
        L.orc_glu.argtypes = [C.c_float, C.c_float, C.c_int]
        L.orc_classify.restype = C.c_uint32
    return _lib


def ref_lib_path() -> str | None:
    """Where oracle/Makefile put the reference's own int4_affine_gemv.c; None if it was not built."""
    path = os.path.join(_HERE, "_ref", "libshrike_ref.so")
    return path if os.path.exists(path) else None


def ref_lib() -> C.CDLL | None:
    """Loads that library (only the one CPU test that compares against it does)."""
    path = ref_lib_path()
    return C.CDLL(path) if path else None


def _p(a: np.ndarray | None):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_void_p)


def expert_offsets(d: int, f: int, bits: int = 4, additive_biases: bool = False):
    off, stride = Offsets(), C.c_uint64()
    lib().orc_expert_offsets(C.c_uint32(d), C.c_uint32(f), C.c_uint32(bits),
                             C.c_int(int(additive_biases)), C.byref(off), C.byref(stride))
    return off, stride.value


def int4_affine_gemv(w, s, b, x, rows, n, meta=META_BF16):
    out = np.empty(rows, np.float32)
    lib().orc_int4_affine_gemv(_p(w), _p(s), _p(b), C.c_int(meta), _p(x),
                               C.c_size_t(rows), C.c_size_t(n), _p(out))
    return out


def affine_gemv(w, s, b, x, rows, n, bits, meta=META_BF16):
    out = np.empty(rows, np.float32)
    lib().orc_affine_gemv(_p(w), _p(s), _p(b), C.c_int(meta), C.c_int(bits), _p(x),
                          C.c_size_t(rows), C.c_size_t(n), _p(out))
    return out


def affine_gemv_f64(w, s, b, x, rows, n, bits, meta=META_BF16):
    out = np.empty(rows, np.float64)
    lib().orc_affine_gemv_f64(_p(w), _p(s), _p(b), C.c_int(meta), C.c_int(bits), _p(x),
                              C.c_size_t(rows), C.c_size_t(n), _p(out))
    return out


def ref_int4_affine_gemv(w, s, b, x, rows, n):
    """Calls the reference's compiled shrike_int4_affine_gemv (bf16 metadata only)."""
    R = ref_lib()
    if R is None:
        raise FileNotFoundError("oracle/_ref/libshrike_ref.so is not built")
    out = np.empty(rows, np.float32)
    R.shrike_int4_affine_gemv(_p(w), _p(s), _p(b), _p(x), C.c_size_t(rows), C.c_size_t(n), _p(out))
    return out


def cpu_expert_ffn_accumulate(blob, off, x, d, f, route_weight, out, bits=4, meta=META_BF16):
    scratch = np.empty(2 * f + d, np.float32)
    lib().orc_cpu_expert_ffn_accumulate(_p(blob), C.byref(off), C.c_int(meta), C.c_int(bits),
                                        _p(x), C.c_uint32(d), C.c_uint32(f),
                                        C.c_float(route_weight), _p(scratch), _p(out))
    return out


def _base_array(blobs):
    """blobs: list of uint8 arrays or None (sentinel) -> (ctypes array of pointers, keepalive)."""
    arr = (C.c_void_p * len(blobs))()
    for i, b in enumerate(blobs):
        arr[i] = None if b is None else b.ctypes.data
    return arr


def moe_phase1(blobs, off, x_f16, d, f, bits=4, meta=META_BF16, act=ACT_SILU,
               additive_biases=False, acts=None):
    k = len(blobs)
    if acts is None:
        acts = np.zeros(k * f, np.uint16)
    lib().orc_moe_phase1(_base_array(blobs), C.byref(off), C.c_int(meta), C.c_int(bits),
                         C.c_int(act), C.c_int(int(additive_biases)), _p(x_f16),
                         C.c_uint32(d), C.c_uint32(f), C.c_uint32(k), _p(acts))
    return acts


def moe_phase2(blobs, off, acts, routing_w_f16, residual_f16, d, f, bits=4, meta=META_BF16,
               additive_biases=False, hidden_f16=None):
    k = len(blobs)
    y = np.empty(d, np.uint16)
    lib().orc_moe_phase2(_base_array(blobs), C.byref(off), C.c_int(meta), C.c_int(bits),
                         C.c_int(int(additive_biases)), _p(acts), _p(routing_w_f16),
                         _p(residual_f16), C.c_uint32(d), C.c_uint32(f), C.c_uint32(k),
                         _p(y), _p(hidden_f16))
    return y


def shared_expert(gate, up, down, x_f16, d, f, bits=4, meta=META_BF16, act=ACT_SILU,
                  scalar_gate_f16=None):
    """gate/up/down: (w, s, b) tuples of numpy arrays."""
    keep = []

    def proj(t):
        p = Proj(t[0].ctypes.data, t[1].ctypes.data, t[2].ctypes.data)
        keep.append(t)
        return p
    g, u, dn = proj(gate), proj(up), proj(down)
    h1 = np.empty(d, np.uint16)
    lib().orc_shared_expert(C.byref(g), C.byref(u), C.byref(dn), C.c_int(meta), C.c_int(bits),
                            C.c_int(act), _p(x_f16), C.c_uint32(d), C.c_uint32(f),
                            _p(scalar_gate_f16), _p(h1))
    return h1


def shared_gate_up(gate, up, x_f16, d, f, bits=4, meta=META_BF16):
    g = Proj(gate[0].ctypes.data, gate[1].ctypes.data, gate[2].ctypes.data)
    u = Proj(up[0].ctypes.data, up[1].ctypes.data, up[2].ctypes.data)
    go, uo = np.empty(f, np.uint16), np.empty(f, np.uint16)
    lib().orc_shared_gate_up(C.byref(g), C.byref(u), C.c_int(meta), C.c_int(bits), _p(x_f16),
                             C.c_uint32(d), C.c_uint32(f), _p(go), _p(uo))
    return go, uo


def shared_down(down, gate_f16, up_f16, d, f, bits=4, meta=META_BF16, act=ACT_SILU, scalar_gate_f16=None):
    dn = Proj(down[0].ctypes.data, down[1].ctypes.data, down[2].ctypes.data)
    h1 = np.empty(d, np.uint16)
    lib().orc_shared_down(C.byref(dn), C.c_int(meta), C.c_int(bits), C.c_int(act), _p(gate_f16),
                          _p(up_f16), C.c_uint32(d), C.c_uint32(f), _p(scalar_gate_f16), _p(h1))
    return h1


def shared_scalar_gate_rows(gate_proj, x_f16, rows, d, x_stride=None, meta=META_BF16):
    """gate_proj: (w u8[d], s u16[d/64], b u16[d/64]) of the one 8-bit gate row; returns fp16 bits[rows]."""
    out = np.empty(rows, np.uint16)
    lib().orc_shared_scalar_gate_rows(_p(gate_proj[0]), _p(gate_proj[1]), _p(gate_proj[2]), C.c_int(meta), _p(x_f16),
                                      C.c_uint32(d if x_stride is None else x_stride), C.c_uint32(rows),
                                      C.c_uint32(d), _p(out))
    return out


def sigmoid_scalar_mul_rows(y_f16, gate_f16, d, rows):
    """In place on y (fp16 bits [rows, d])."""
    lib().orc_sigmoid_scalar_mul_rows(_p(y_f16), _p(gate_f16), C.c_uint32(d), C.c_uint32(rows))
    return y_f16


def router_logits(weights, scales, biases, kind, hidden_f16, eff_scale_bf16, num_experts, d,
                  meta=META_BF16):
    out = np.empty(num_experts, np.float32)
    lib().orc_router_logits(_p(weights), _p(scales), _p(biases), C.c_int(kind), C.c_int(meta),
                            _p(hidden_f16), _p(eff_scale_bf16), C.c_uint32(num_experts),
                            C.c_uint32(d), _p(out))
    return out


def router_select(logits, per_expert_scale_bf16, bias_bf16, top_k, sigmoid=False, scaling=1.0):
    n = logits.shape[0]
    idx = np.empty(top_k, np.uint32)
    w = np.empty(top_k, np.uint16)
    lib().orc_router_select(_p(logits), _p(per_expert_scale_bf16), _p(bias_bf16),
                            C.c_uint32(n), C.c_uint32(top_k), C.c_int(int(sigmoid)),
                            C.c_float(scaling), _p(idx), _p(w))
    return idx, w


def classify(topk, residency_u64, num_experts):
    k = topk.shape[0]
    hc, mc = np.zeros(1, np.uint32), np.zeros(1, np.uint32)
    hp, mp, me = (np.zeros(k, np.uint32) for _ in range(3))
    rs = np.zeros(k, np.uint32)
    lib().orc_classify(_p(topk), _p(residency_u64), C.c_uint32(k), C.c_uint32(num_experts),
                       _p(hc), _p(hp), _p(mc), _p(mp), _p(me), _p(rs))
    return dict(hit_count=int(hc[0]), miss_count=int(mc[0]), hit_positions=hp[:hc[0]].copy(),
                miss_positions=mp[:mc[0]].copy(), miss_experts=me[:mc[0]].copy(),
                resolved_slots=rs)


def prefill_reduce(partials_f16, weights_f16, t, top_k, d):
    h2 = np.empty(t * d, np.uint16)
    lib().orc_prefill_reduce(_p(partials_f16), _p(weights_f16), C.c_uint32(t), C.c_uint32(top_k),
                             C.c_uint32(d), _p(h2))
    return h2


def residual_add_f16(hidden, delta):
    lib().orc_residual_add_f16(_p(hidden), _p(delta), C.c_size_t(hidden.shape[0]))
    return hidden


def residual_add_rmsnorm_bf16w(hidden, delta, weight_bf16, eps):
    """In place on `hidden` (fp16 bits); returns the normalised row (fp16 bits). delta None: rmsnorm only."""
    out = np.empty_like(hidden)
    lib().orc_residual_add_rmsnorm_bf16w(_p(hidden), _p(delta) if delta is not None else None, _p(weight_bf16), _p(out),
                                         C.c_uint32(hidden.shape[0]), C.c_float(eps))
    return out


def cpu_layer_fp32(blobs, route_weights, off, x_f32, d, f, threads, bits=4, meta=META_BF16):
    out = np.zeros(d, np.float32)
    rw = np.ascontiguousarray(route_weights, np.float32)
    lib().orc_cpu_layer_fp32(_base_array(blobs), _p(rw), C.c_uint32(len(blobs)), C.byref(off),
                             C.c_int(meta), C.c_int(bits), _p(x_f32), C.c_uint32(d),
                             C.c_uint32(f), C.c_uint32(threads), _p(out))
    return out


# ---------------------------------------------------------------- whole layer (composition)

def moe_decode_layer(x_f16, hidden_f16, router, pool_blobs, residency_u64, off, d, f, top_k,
                     shared=None, bits=4, meta=META_BF16, act=ACT_SILU, sigmoid=False,
                     scaling=1.0, additive_biases=False):
    """One decode layer in the order the reference's runner encodes it
    (sources/Shrike/Runtime/Inference/RealForwardRunner.swift:2834-2901, :5520-5560):
    router -> select -> classify -> shared expert (h1) -> phase 1 -> phase 2 with
    residual = h1. `router` is a dict(weights, scales, biases, kind, eff_scale, expert_scale,
    bias); `pool_blobs[cell]` are the resident blobs; `shared` = dict(gate, up, down, f,
    bits, scalar_gate) or None (residual = 0)."""
    ne = router["expert_scale"].shape[0]
    logits = router_logits(router["weights"], router.get("scales"), router.get("biases"),
                           router["kind"], x_f16, router["eff_scale"], ne, d,
                           meta=router.get("meta", META_BF16))
    idx, w = router_select(logits, router["expert_scale"], router["bias"], top_k, sigmoid, scaling)
    cls = classify(idx, residency_u64, ne)
    blobs = [None if s == 0xFFFFFFFF else pool_blobs[int(s)] for s in cls["resolved_slots"]]
    if shared is not None:
        h1 = shared_expert(shared["gate"], shared["up"], shared["down"], x_f16, d, shared["f"],
                           bits=shared.get("bits", bits), meta=meta, act=act,
                           scalar_gate_f16=shared.get("scalar_gate"))
    else:
        h1 = np.zeros(d, np.uint16)
    acts = moe_phase1(blobs, off, x_f16, d, f, bits=bits, meta=meta, act=act,
                      additive_biases=additive_biases)
    hidden = hidden_f16.copy()
    y = moe_phase2(blobs, off, acts, w, h1, d, f, bits=bits, meta=meta,
                   additive_biases=additive_biases, hidden_f16=hidden)
    return dict(logits=logits, indices=idx, weights=w, classify=cls, h1=h1, acts=acts, y=y,
                hidden=hidden)


# ------------------------------------------------------------------ prefill (composition)

def prefill_router(router, hidden_f16, query_count, d, top_k, stride=None, sigmoid=False, scaling=1.0):
    """The router for query_count tokens, token by token with the decode functions
    (sources/Shrike/Metal/Prefill/prefill.metal:369-563 computes the same per token).
    Returns (indices u32[T*K], weights f16 bits[T*K], logits f32[T, E])."""
    stride = d if stride is None else stride
    ne = router["expert_scale"].shape[0]
    idx = np.empty(query_count * top_k, np.uint32)
    w = np.empty(query_count * top_k, np.uint16)
    logits = np.empty((query_count, ne), np.float32)
    for t in range(query_count):
        x = np.ascontiguousarray(hidden_f16[t * stride:t * stride + d])
        logits[t] = router_logits(router["weights"], router.get("scales"), router.get("biases"), router["kind"], x,
                                  router["eff_scale"], ne, d, meta=router.get("meta", META_BF16))
        i, ww = router_select(logits[t], router["expert_scale"], router["bias"], top_k, sigmoid, scaling)
        idx[t * top_k:(t + 1) * top_k], w[t * top_k:(t + 1) * top_k] = i, ww
    return idx, w, logits


def prefill_pair_partial(blob, off, x_f16, d, f, bits=4, meta=META_BF16, act=ACT_SILU, additive_biases=False):
    """One (token, expert) pair's partial row as the reference's scalar model computes it
    (tests/Shrike/Core/Kernels/Prefill/PrefillGroupedRoutedMoETests.swift:368-473): gate and up
    in fp32, act rounded to fp16, down in fp32, the row rounded to fp16. A phase-2 pass with
    weight 1 and residual 0 gives exactly that rounding."""
    acts = moe_phase1([blob], off, x_f16, d, f, bits, meta, act, additive_biases)
    one = np.array([0x3C00], np.uint16)
    zero = np.zeros(d, np.uint16)
    return moe_phase2([blob], off, acts, one, zero, d, f, bits, meta, additive_biases)
