"""GPU parity: the decode kernels behind the C ABI against the CPU oracle on the same
seeded bytes. Routing indices, residency lists and logits are compared bit for bit;
FFN outputs within max-abs 2e-3 / relative 1e-3 (|a-b| <= 2e-3 + 1e-3*|b|)."""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle as O
from shrike_amd import capi
from shrike_amd import host as HL
from shrike_amd import synth as S
from harness import runners
from tests.helpers import Layer, assert_ffn_close, assert_rel_close, f16

pytestmark = pytest.mark.gpu
SENT = 0xFFFFFFFF


class DeviceLayer:
    """Uploads a Layer: every expert resident in a pool, cell = a permutation of the expert id."""

    def __init__(self, rt, layer: Layer, cells=None, chunk_bytes=0, resident=None, moe_kwargs=None, pool=None):
        self.rt, self.L = rt, layer
        L = layer
        cells = cells or L.ne
        self.pool = pool or rt.ExpertPool(cells, L.stride, L.ne, chunk_bytes)
        self.cell_of = {}
        resident = range(L.ne) if resident is None else resident
        for i, e in enumerate(resident):
            cell = (i * 7 + 3) % cells if cells == L.ne and np.gcd(7, cells) == 1 else i
            self.pool.upload(cell, L.blobs[e])
            self.pool.publish(e, cell, capi.RESIDENT)
            self.cell_of[e] = cell
        self.off, stride = rt.expert_offsets(L.d, L.f, L.bits, L.additive)
        assert stride == L.stride
        kw = dict(routed_bits=L.bits, router_bits=L.router_bits, meta=L.meta)
        kw.update(moe_kwargs or {})
        self.moe = rt.MoE(L.d, L.f, L.ne, L.k, **kw)
        dev = rt.dev
        self.router_w = dev(L.router_w)
        self.router_s = dev(L.router_s) if L.router_s is not None else None
        self.router_b = dev(L.router_b) if L.router_b is not None else None
        self.eff_scale, self.expert_scale, self.logit_bias = dev(L.eff_scale), dev(L.expert_scale), dev(L.logit_bias)
        self.x, self.hidden = dev(L.x), dev(L.hidden)
        self.out_idx, self.out_w = rt.empty(4 * 8), rt.empty(2 * 8)
        self.resolved = rt.empty(4 * 8)
        self.hit_count, self.miss_count = rt.empty(4), rt.empty(4)
        self.hit_pos, self.miss_pos, self.miss_exp = rt.empty(32), rt.empty(32), rt.empty(32)
        self.acts = rt.empty(2 * L.k * L.f)
        self.y, self.h1 = rt.empty(2 * L.d), rt.empty(2 * L.d)
        if L.shared_f:
            self.shared = {n: tuple(dev(t) for t in L.shared[n]) for n in ("gate", "up", "down")}
            self.shared_scratch = rt.empty(2 * 2 * L.shared_f)

    def pool_blobs(self):
        """cell -> blob, for the oracle."""
        out = {}
        for e, c in self.cell_of.items():
            out[c] = self.L.blobs[e]
        return out

    def residency_words(self):
        return np.array([self.pool.entry(e) for e in range(self.L.ne)], np.uint64)

    def layer_args(self):
        L = self.L
        a = capi.DecodeLayerArgs()
        a.router_weights = self.router_w.ptr
        a.router_scales = self.router_s.ptr if self.router_s else None
        a.router_biases = self.router_b.ptr if self.router_b else None
        a.effective_scale, a.per_expert_scale, a.logit_bias = self.eff_scale.ptr, self.expert_scale.ptr, self.logit_bias.ptr
        a.pool, a.pool_slot_stride, a.residency = self.pool.bases, self.pool.stride, self.pool.table
        a.offsets = self.off
        if L.shared_f:
            for name in ("gate", "up", "down"):
                w, s, b = self.shared[name]
                setattr(a, f"shared_{name}", capi.Projection(w.ptr, s.ptr, b.ptr))
            a.shared_bits, a.shared_f = L.shared_bits, L.shared_f
            a.shared_scratch = self.shared_scratch.ptr
        a.x, a.hidden, a.y = self.x.ptr, self.hidden.ptr, self.y.ptr
        a.out_indices, a.out_weights = self.out_idx.ptr, self.out_w.ptr
        a.resolved_slots, a.hit_count, a.hit_positions = self.resolved.ptr, self.hit_count.ptr, self.hit_pos.ptr
        a.miss_count, a.miss_positions, a.miss_experts = self.miss_count.ptr, self.miss_pos.ptr, self.miss_exp.ptr
        a.acts, a.h1 = self.acts.ptr, self.h1.ptr
        return a


def oracle_layer(L: Layer, dl: DeviceLayer, **kw):
    shared = None
    if L.shared_f:
        shared = dict(gate=L.shared["gate"], up=L.shared["up"], down=L.shared["down"], f=L.shared_f,
                      bits=L.shared_bits)
    return O.moe_decode_layer(L.x, L.hidden, L.router_dict(), dl.pool_blobs(), dl.residency_words(),
                              L.oracle_offsets(), L.d, L.f, L.k, shared=shared, bits=L.bits, meta=L.meta,
                              additive_biases=L.additive, **kw)


# --------------------------------------------------------------------------- router

@pytest.mark.parametrize("router_bits", [0, 8, 4])
@pytest.mark.parametrize("ne,d,k", [(256, 2048, 8), (32, 2880, 4), (256, 2304, 8), (16, 128, 8), (5, 64, 3)])
def test_router_logits_and_indices_bit_exact(gpu, router_bits, ne, d, k):
    L = Layer(0x5EED0002 + router_bits, d, 64, ne, k, router_bits=router_bits)
    L.logit_bias = S.f32_to_bf16_bits(L.tree.key("bias").normal(ne, std=0.01))
    L.expert_scale = S.f32_to_bf16_bits(L.tree.key("escale").uniform(0.6, 1.4, ne))
    L.eff_scale = S.f32_to_bf16_bits(L.tree.key("eff").uniform(0.5, 1.5, d))
    dl = DeviceLayer(gpu, L, resident=[])
    dl.moe.encode_router(dl.router_w, dl.router_s, dl.router_b, dl.x, dl.eff_scale, dl.expert_scale,
                         dl.logit_bias, dl.out_idx, dl.out_w, ne, d, k)
    logits = dl.moe.logits(ne)
    ref_logits = O.router_logits(L.router_w, L.router_s, L.router_b, router_bits, L.x, L.eff_scale, ne, d)
    assert np.array_equal(logits.view(np.uint32), ref_logits.view(np.uint32)), "router logits differ in bits"
    idx = dl.out_idx.download(np.uint32, k)
    w = dl.out_w.download(np.uint16, k)
    ref_idx, ref_w = O.router_select(ref_logits, L.expert_scale, L.logit_bias, k)
    assert np.array_equal(idx, ref_idx)
    assert np.max(np.abs(f16(w) - f16(ref_w))) <= 1e-3  # reference holds weights to 5e-3 (RouterTopKTests.swift:43)
    # the select stage alone, on the device's own logits
    idx2, _ = O.router_select(logits, L.expert_scale, L.logit_bias, k)
    assert np.array_equal(idx, idx2)


def test_router_ties_go_to_the_lower_index(gpu):
    # identical rows -> identical logits: selection must be experts 0..k-1 in order
    ne, d, k = 64, 256, 8
    L = Layer(7, d, 64, ne, k)
    L.router_w[:] = L.router_w[0]
    dl = DeviceLayer(gpu, L, resident=[])
    dl.moe.encode_router(dl.router_w, None, None, dl.x, dl.eff_scale, dl.expert_scale, dl.logit_bias,
                         dl.out_idx, dl.out_w, ne, d, k)
    assert dl.out_idx.download(np.uint32, k).tolist() == list(range(k))
    assert np.allclose(f16(dl.out_w.download(np.uint16, k)), 1.0 / k, atol=1e-3)


def test_router_sigmoid_scores(gpu):
    ne, d, k = 256, 2304, 8
    L = Layer(0x516, d, 64, ne, k, router_bits=8)
    L.logit_bias = S.f32_to_bf16_bits(L.tree.key("corr").uniform(-0.2, 0.2, ne))
    dl = DeviceLayer(gpu, L, resident=[], moe_kwargs=dict(sigmoid=True, scaling=2.446))
    dl.moe.encode_router(dl.router_w, dl.router_s, dl.router_b, dl.x, dl.eff_scale, dl.expert_scale,
                         dl.logit_bias, dl.out_idx, dl.out_w, ne, d, k)
    logits = dl.moe.logits(ne)
    ref_idx, ref_w = O.router_select(logits, L.expert_scale, L.logit_bias, k, sigmoid=True, scaling=2.446)
    # sigmoid selection compares sigmoid(logit)+bias: device expf and libm expf may differ in the last
    # bit, so the selection is checked on scores recomputed here with a gap guard.
    idx = dl.out_idx.download(np.uint32, k)
    s = 1.0 / (1.0 + np.exp(-logits.astype(np.float64))) + S.bf16_bits_to_f32(L.logit_bias)
    order = np.lexsort((np.arange(ne), -s))
    gap = s[order[k - 1]] - s[order[k]]
    if gap > 1e-6:
        assert np.array_equal(np.sort(idx), np.sort(order[:k].astype(np.uint32)))
        assert np.array_equal(idx, ref_idx)
    assert np.max(np.abs(f16(dl.out_w.download(np.uint16, k)) - f16(ref_w))) <= 2e-3


# ------------------------------------------------------------------------- classify

def test_classify_truth_table_and_spec_args(gpu):
    ne, k = 16, 8
    L = Layer(3, 64, 64, ne, k)
    dl = DeviceLayer(gpu, L, resident=[])
    words = np.full(ne, (0 << 32) | SENT, np.uint64)
    words[2] = (2 << 32) | 5          # resident at cell 5
    words[3] = (1 << 32) | 6          # loading: a miss
    words[4] = (2 << 32) | SENT       # resident but no slot: a miss
    words[9] = (2 << 32) | 0
    table = gpu.dev(words)
    topk = np.array([2, 3, 4, 9, 0, 200, 2, 9], np.uint32)  # 200 clamps to ne-1 (empty)
    weights = S.f32_to_f16_bits(np.linspace(0.3, 0.05, k).astype(np.float32))
    pred = np.arange(100, 100 + k, dtype=np.uint32)
    spec, readback = gpu.empty(48), gpu.empty(4 * (2 + 5 * k))
    full = [256, 1, 1, 13, 7, 1, 256, 1, 1, 13, 7, 1]
    dl.moe.encode_residency_classification(gpu.dev(topk), table, dl.hit_count, dl.hit_pos, dl.miss_count,
                                           dl.miss_pos, dl.miss_exp, dl.resolved, k, ne, full_grids=full,
                                           spec_args=spec, host_readback=readback, tag=0x1234,
                                           topk_weights=gpu.dev(weights), predicted=gpu.dev(pred))
    ref = O.classify(topk, words, ne)
    hits, misses = dl.hit_count.download(np.uint32, 1)[0], dl.miss_count.download(np.uint32, 1)[0]
    assert (hits, misses) == (ref["hit_count"], ref["miss_count"]) == (4, 4)
    assert np.array_equal(dl.hit_pos.download(np.uint32, hits), ref["hit_positions"])
    assert np.array_equal(dl.miss_pos.download(np.uint32, misses), ref["miss_positions"])
    assert np.array_equal(dl.miss_exp.download(np.uint32, misses), ref["miss_experts"])
    assert np.array_equal(dl.resolved.download(np.uint32, k), ref["resolved_slots"])
    # a miss: phase 1 keeps the full grid, phase 2 gets a zero-width grid, the fixup the full ones
    # (GPUExpertResidencyTests.swift:16-22)
    assert spec.download(np.uint32, 12).tolist() == [256, 1, 1, 0, 1, 1, 256, 1, 1, 13, 7, 1]
    rb = readback.download(np.uint32, 2 + 5 * k)
    t = 0x1234 << 16
    assert rb[0] == t | 4 and rb[1] == t | 4
    assert rb[2:2 + k].tolist() == [t | min(int(e), ne - 1) for e in topk]
    assert rb[2 + k:2 + 2 * k].tolist() == [t | int(b) for b in weights]
    assert rb[2 + 2 * k:2 + 3 * k].tolist() == [t | int(p) for p in ref["hit_positions"]] + [t] * 4
    assert rb[2 + 3 * k:2 + 4 * k].tolist() == [t | int(p) for p in ref["miss_positions"]] + [t] * 4
    assert rb[2 + 4 * k:].tolist() == [t | int(p) for p in pred]
    # all hit
    topk2 = np.array([2, 9, 2, 9, 2, 9, 2, 9], np.uint32)
    dl.moe.encode_residency_classification(gpu.dev(topk2), table, dl.hit_count, dl.hit_pos, dl.miss_count,
                                           dl.miss_pos, dl.miss_exp, dl.resolved, k, ne, full_grids=full,
                                           spec_args=spec)
    assert spec.download(np.uint32, 12).tolist() == [256, 1, 1, 13, 7, 1, 0, 1, 1, 0, 1, 1]
    assert dl.resolved.download(np.uint32, k).tolist() == [5, 0, 5, 0, 5, 0, 5, 0]


# --------------------------------------------------------------------- phase 1 / 2

SHAPES = [  # d, f
    (2048, 512), (128, 64), (192, 320), (704, 192), (2880, 2880), (2304, 1024), (4096, 256),
    # 4-bit rows that end in a step of half chunks behind one, two and three whole steps (and the 8-bit rows of the same sizes)
    (2304, 4352), (128, 6400), (3072, 2112)]


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("meta", [S.META_BF16, S.META_F16])
@pytest.mark.parametrize("d,f", SHAPES)
def test_phase1_phase2_against_oracle(gpu, bits, meta, d, f):
    if max(d, f) * bits // 128 > 256:
        pytest.skip("row longer than four wave loads")
    k, ne = 8, 8
    if d * f > 4_000_000:
        k, ne = 4, 4
    check_phase1_phase2(gpu, bits, meta, d, f, k, ne, 0x5EED0000 + d + f + bits)


def _swept_shapes():
    """Ninety-six shapes drawn once from a fixed seed: hidden and intermediate sizes any multiple of 64 up to 2,560
    (rows of 1 to 160 sixteen-byte chunks: every chunks-per-lane count, whole and ragged waves, rows shorter than
    a wave load), 1 to 8 routed positions, both code widths and both metadata types."""
    rng = np.random.default_rng(0x5EED5EED)
    out = []
    for _ in range(96):
        d, f = (int(64 * rng.integers(1, 41)) for _ in range(2))
        out.append((d, f, int(rng.integers(1, 9)), int(rng.choice([4, 8])), int(rng.choice([S.META_BF16, S.META_F16]))))
    return out


@pytest.mark.parametrize("d,f,k,bits,meta", _swept_shapes())
def test_phase1_phase2_shape_sweep(gpu, d, f, k, bits, meta):
    check_phase1_phase2(gpu, bits, meta, d, f, k, k, 0x5EED1000 + d * 41 + f + k)


def check_phase1_phase2(gpu, bits, meta, d, f, k, ne, seed):
    L = Layer(seed, d, f, ne, k, bits=bits, meta=meta)
    dl = DeviceLayer(gpu, L)
    resolved = np.array([dl.cell_of[e] for e in range(k)], np.uint32)
    resolved[k - 1] = SENT  # one sentinel position: its acts must stay untouched, its partial must be zero
    d_res = gpu.dev(resolved)
    acts0 = S.f32_to_f16_bits(np.full(k * f, 0.25, np.float32))
    dl.acts.upload(acts0)
    dl.moe.encode_spec_phase1(dl.pool, d_res, dl.off, dl.x, dl.acts, d, f, k)
    acts = dl.acts.download(np.uint16, k * f)
    blobs = [None if s == SENT else dl.pool_blobs()[int(s)] for s in resolved]
    ref_acts = O.moe_phase1(blobs, L.oracle_offsets(), L.x, d, f, bits=bits, meta=meta, acts=acts0.copy())
    assert np.array_equal(acts[(k - 1) * f:], acts0[(k - 1) * f:]), "sentinel position was written"
    assert_ffn_close(acts, ref_acts, "phase-1 acts")

    w = S.f32_to_f16_bits(L.tree.key("w").uniform(0.05, 0.3, k))
    residual = S.activations_f16(L.tree, "residual", d)
    hidden = L.hidden.copy()
    # phase 2 from the ORACLE's acts so the comparison isolates the down matvec + combine
    dl.acts.upload(ref_acts)
    dl.moe.encode_spec_phase2(dl.pool, d_res, dl.off, dl.acts, gpu.dev(w), gpu.dev(residual), dl.y,
                              dl.hidden, d, f, k)
    ref_y = O.moe_phase2(blobs, L.oracle_offsets(), ref_acts, w, residual, d, f, bits=bits, meta=meta,
                         hidden_f16=hidden)
    y = dl.y.download(np.uint16, d)
    assert_ffn_close(y, ref_y, "phase-2 y")
    # hidden += y is exact given y (moe.metal:889-893)
    got_hidden = dl.hidden.download(np.uint16, d)
    expect_hidden = O.residual_add_f16(L.hidden.copy(), y)
    assert np.array_equal(got_hidden, expect_hidden)


@pytest.mark.parametrize("bits,d,f,k", [(4, 2048, 512, 8), (8, 256, 128, 4), (4, 2880, 384, 3)])
def test_argument_buffer_operators(gpu, bits, d, f, k):
    """encodeRoutedPersistentPhase1U16Load / ...SubsetU16Load / ...Phase2Reduce: the route's blobs named by a device
    array of pointers. Against the oracle, and byte for byte the pool operators' results over the same blobs."""
    L = Layer(0x5EED0A00 + d + bits, d, f, k + 2, k, bits=bits)
    dl = DeviceLayer(gpu, L)
    order = [(3 * p + 1) % (k + 2) for p in range(k)]  # position p's expert
    cells = np.array([dl.cell_of[e] for e in order], np.uint32)
    arg = dl.moe.make_routed_argument_buffer([dl.pool.cell_ptr(int(c)) for c in cells])
    blobs = [dl.pool_blobs()[int(c)] for c in cells]
    acts0 = S.f32_to_f16_bits(np.full(k * f, 0.25, np.float32))
    # all positions
    dl.acts.upload(acts0)
    dl.moe.encode_routed_persistent_phase1(arg, dl.off, dl.x, dl.acts, d, f, k)
    acts = dl.acts.download(np.uint16, k * f)
    ref_acts = O.moe_phase1(blobs, L.oracle_offsets(), L.x, d, f, bits=bits, acts=acts0.copy())
    assert_ffn_close(acts, ref_acts, "argument-buffer phase-1 acts")
    dl.acts.upload(acts0)
    dl.moe.encode_spec_phase1(dl.pool, gpu.dev(cells), dl.off, dl.x, dl.acts, d, f, k)
    assert np.array_equal(acts, dl.acts.download(np.uint16, k * f))
    # a subset: listed positions only, in list order, an entry past top_k skipped
    active = np.array([k - 1, 0, k + 5], np.uint32)
    dl.acts.upload(acts0)
    dl.moe.encode_routed_persistent_phase1(arg, dl.off, dl.x, dl.acts, d, f, k, active_slots=gpu.dev(active), active_count=3)
    sub = dl.acts.download(np.uint16, k * f)
    for p in range(k):
        want = acts if p in (0, k - 1) else acts0
        assert np.array_equal(sub[p * f:(p + 1) * f], want[p * f:(p + 1) * f]), p
    dl.acts.upload(acts0)
    dl.moe.encode_routed_persistent_phase1(arg, dl.off, dl.x, dl.acts, d, f, k, active_slots=gpu.dev(active), active_count=0)
    assert np.array_equal(dl.acts.download(np.uint16, k * f), acts0)
    # phase 2 over the argument buffer
    w = S.f32_to_f16_bits(L.tree.key("w").uniform(0.05, 0.3, k))
    residual = S.activations_f16(L.tree, "residual", d)
    dl.acts.upload(ref_acts)
    dw, dr = gpu.dev(w), gpu.dev(residual)
    dl.moe.encode_routed_persistent_phase2(arg, dl.off, dl.acts, dw, dr, dl.y, dl.hidden, d, f, k)
    y, hidden = dl.y.download(np.uint16, d), dl.hidden.download(np.uint16, d)
    ref_y = O.moe_phase2(blobs, L.oracle_offsets(), ref_acts, w, residual, d, f, bits=bits, hidden_f16=L.hidden.copy())
    assert_ffn_close(y, ref_y, "argument-buffer phase-2 y")
    assert np.array_equal(hidden, O.residual_add_f16(L.hidden.copy(), y))
    dl.hidden.upload(L.hidden)
    dl.moe.encode_spec_phase2(dl.pool, gpu.dev(cells), dl.off, dl.acts, dw, dr, dl.y, dl.hidden, d, f, k)
    assert np.array_equal(y, dl.y.download(np.uint16, d)) and np.array_equal(hidden, dl.hidden.download(np.uint16, d))
    # an unbound argument buffer is an error, not a fault
    with pytest.raises(capi.ShrikeError, match="argument buffer"):
        dl.moe.encode_routed_persistent_phase1(None, dl.off, dl.x, dl.acts, d, f, k)
    with pytest.raises(capi.ShrikeError, match="activeCount"):
        dl.moe.encode_routed_persistent_phase1(arg, dl.off, dl.x, dl.acts, d, f, k, active_slots=gpu.dev(active), active_count=9)


def test_phase2_fallback_cells_and_indirect_zero_grid(gpu):
    d, f, k = 256, 128, 4
    L = Layer(11, d, f, k, k)
    dl = DeviceLayer(gpu, L)
    cells = np.array([dl.cell_of[e] for e in range(k)], np.uint32)
    resolved = cells.copy()
    resolved[1] = SENT
    acts = O.moe_phase1([dl.pool_blobs()[int(c)] for c in cells], L.oracle_offsets(), L.x, d, f)
    dl.acts.upload(acts)
    w = S.f32_to_f16_bits(np.full(k, 0.25, np.float32))
    residual = np.zeros(d, np.uint16)
    dw, dr = gpu.dev(w), gpu.dev(residual)
    # fallback supplies the missing cell (moe.metal:1037-1038)
    dl.moe.encode_spec_phase2(dl.pool, gpu.dev(resolved), dl.off, dl.acts, dw, dr, dl.y, None, d, f, k,
                              fallback_cells=gpu.dev(cells))
    ref = O.moe_phase2([dl.pool_blobs()[int(c)] for c in cells], L.oracle_offsets(), acts, w, residual, d, f)
    assert_ffn_close(dl.y.download(np.uint16, d), ref, "fallback")
    # zero-width indirect grid: nothing is written
    dl.y.upload(np.full(d, 0x3C00, np.uint16))
    dl.moe.encode_spec_phase2(dl.pool, gpu.dev(cells), dl.off, dl.acts, dw, dr, dl.y, None, d, f, k,
                              indirect=gpu.dev(np.array([0, 1, 1], np.uint32)))
    assert np.all(dl.y.download(np.uint16, d) == 0x3C00)


def test_event_gated_status_word(gpu):
    d, f, k = 128, 64, 2
    L = Layer(12, d, f, k, k)
    dl = DeviceLayer(gpu, L, moe_kwargs=dict(event_gated=True))
    cells = gpu.dev(np.array([dl.cell_of[e] for e in range(k)], np.uint32))
    residual = S.activations_f16(L.tree, "r", d)
    w = gpu.dev(S.f32_to_f16_bits(np.full(k, 0.5, np.float32)))
    failed = gpu.dev(np.array([2], np.uint32))  # a failed batch (moe.metal:36-39)
    acts0 = np.full(k * f, 0x1234, np.uint16)
    dl.acts.upload(acts0)
    dl.moe.encode_spec_phase1(dl.pool, cells, dl.off, dl.x, dl.acts, d, f, k, io_status=failed)
    assert np.array_equal(dl.acts.download(np.uint16, k * f), acts0)
    dl.moe.encode_spec_phase2(dl.pool, cells, dl.off, dl.acts, w, gpu.dev(residual), dl.y, dl.hidden, d, f, k,
                              io_status=failed)
    assert np.array_equal(dl.y.download(np.uint16, d), residual)  # residual written through (:918-921)
    assert np.array_equal(dl.hidden.download(np.uint16, d), O.residual_add_f16(L.hidden.copy(), residual))


def test_closed_form_ffn(gpu):
    """q=0, scale=0: gate = bias*sum(x) = 1, up = 0.5, act = 0.5*silu(1); down bias 1/64 over F=64
    -> each expert returns act; eight experts at 0.125 -> silu(1)*0.5... scaled as the reference's
    known-answer test (MoEFusedFFNTests.swift:17-55, :868-900): gate bias 1/64, up bias 0.5/64,
    down bias 1/64, x = 1, D=128, F=64 -> every output 2/(1+e^-2) within 0.01."""
    d, f, k = 128, 64, 8
    off, stride = S.expert_offsets(d, f, 4)
    blob = np.zeros(stride, np.uint8)

    def put(name, value, count):
        blob[off[name]:off[name] + 2 * count] = np.full(count, S.f32_to_bf16_bits(np.array([value], np.float32))[0],
                                                        np.uint16).view(np.uint8)
    put("gate_b", 1.0 / 64.0, f * (d // 64))
    put("up_b", 0.5 / 64.0, f * (d // 64))
    put("down_b", 1.0 / 64.0, d * (f // 64))
    pool = gpu.ExpertPool(k, stride, k)
    for c in range(k):
        pool.upload(c, blob)
    moe = gpu.MoE(d, f, k, k)
    o, _ = gpu.expert_offsets(d, f, 4)
    x = gpu.dev(S.f32_to_f16_bits(np.ones(d, np.float32)))
    acts, y = gpu.empty(2 * k * f), gpu.empty(2 * d)
    res = gpu.dev(np.arange(k, dtype=np.uint32))
    moe.encode_spec_phase1(pool, res, o, x, acts, d, f, k)
    moe.encode_spec_phase2(pool, res, o, acts, gpu.dev(S.f32_to_f16_bits(np.full(k, 0.125, np.float32))),
                           gpu.dev(np.zeros(d, np.uint16)), y, None, d, f, k)
    # gate = (1/64)*128 = 2, up = (0.5/64)*128 = 1, act = silu(2)*1 = 2/(1+e^-2); down = (1/64)*64*act
    expect = 2.0 / (1.0 + np.exp(-2.0))
    assert np.all(np.abs(f16(y.download(np.uint16, d)) - expect) <= 0.01)
    assert np.all(np.abs(f16(acts.download(np.uint16, k * f)) - expect) <= 2e-3)


# --------------------------------------------------------------------- shared expert

@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("d,fs", [(2048, 512), (2304, 1024), (128, 64), (192, 320)])
def test_shared_expert_against_oracle(gpu, bits, d, fs):
    L = Layer(0x5EED0100 + d + bits, d, 64, 2, 1, shared_f=fs, shared_bits=bits)
    dl = DeviceLayer(gpu, L, resident=[])
    sh = L.shared
    for gate in (None, S.f32_to_f16_bits(np.array([0.3], np.float32))):
        dl.moe.encode_shared_expert(dl.shared["gate"], dl.shared["up"], dl.shared["down"], bits, dl.x,
                                    dl.shared_scratch, dl.h1, d, fs,
                                    scalar_gate=None if gate is None else gpu.dev(gate))
        check_shared_stages(dl, L, gate)


def check_shared_stages(dl, L, gate=None):
    """Each stage against the oracle fed with the device's previous stage (one fp16 rounding per
    comparison), then the whole chain with the reference's relative metric."""
    d, fs, bits, sh = L.d, L.shared_f, L.shared_bits, L.shared
    halves = dl.shared_scratch.download(np.uint16, 2 * fs)
    g_dev, u_dev = halves[:fs].copy(), halves[fs:].copy()
    g_ref, u_ref = O.shared_gate_up(sh["gate"], sh["up"], L.x, d, fs, bits=bits, meta=L.meta)
    assert_ffn_close(g_dev, g_ref, "shared gate rows")
    assert_ffn_close(u_dev, u_ref, "shared up rows")
    h1 = dl.h1.download(np.uint16, d)
    # a gated output is rounded to fp16 twice in a row (dequant_int4.metal:322-329): two fp16 steps
    assert_ffn_close(h1, O.shared_down(sh["down"], g_dev, u_dev, d, fs, bits=bits, meta=L.meta,
                                       scalar_gate_f16=gate), "shared down from the device's gate/up",
                     rel=1e-3 if gate is None else 2e-3)
    assert_rel_close(h1, O.shared_expert(sh["gate"], sh["up"], sh["down"], L.x, d, fs, bits=bits, meta=L.meta,
                                         scalar_gate_f16=gate), "shared expert end to end",
                     tol=1e-3 if gate is None else 2e-3)
    return h1


# ------------------------------------------------------------------------ whole layer

CONFIGS = [
    # name, d, f, E, K, bits, meta, router_bits, shared_f
    ("q35b-a3b-int4-f16meta", 2048, 512, 256, 8, 4, S.META_F16, 0, 512),
    ("q35b-a3b-int4-bf16meta-affine8-router", 2048, 512, 256, 8, 4, S.META_BF16, 8, 512),
    ("gpt-oss-int4", 2880, 2880, 32, 4, 4, S.META_BF16, 0, 0),
    ("gpt-oss-int8", 2880, 2880, 32, 4, 8, S.META_BF16, 0, 0),
    ("kimi-int8", 2304, 1024, 64, 8, 8, S.META_BF16, 8, 1024),
    ("toy", 128, 64, 16, 8, 4, S.META_BF16, 0, 64),
]


# the whole layer against the oracle, element by element: the worst element in fp16 steps of the vector's largest
# magnitude, and the share of elements that may be outside 2e-3 + 1e-3|b| at all
LAYER_WORST_STEPS, LAYER_OUTSIDE_SHARE = 2.0, 0.05


@pytest.mark.parametrize("cfg", CONFIGS, ids=[c[0] for c in CONFIGS])
def test_decode_layer_matches_oracle_and_split_calls(gpu, cfg):
    name, d, f, ne, k, bits, meta, rbits, fs = cfg
    n_blobs = ne if d * f * ne < 600_000_000 else 8
    L = Layer(0x5EED0002, d, f, ne, k, bits=bits, meta=meta, router_bits=rbits, shared_f=fs)
    dl = DeviceLayer(gpu, L)
    dl.moe.encode_decode_layer(dl.layer_args())
    ref = oracle_layer(L, dl)
    idx = dl.out_idx.download(np.uint32, k)
    assert np.array_equal(idx, ref["indices"]), "routing indices differ"
    assert np.array_equal(dl.moe.logits(ne).view(np.uint32), ref["logits"].view(np.uint32))
    assert np.array_equal(dl.resolved.download(np.uint32, k), ref["classify"]["resolved_slots"])
    assert dl.hit_count.download(np.uint32, 1)[0] == k and dl.miss_count.download(np.uint32, 1)[0] == 0
    assert np.max(np.abs(f16(dl.out_w.download(np.uint16, k)) - f16(ref["weights"]))) <= 1e-3
    h1 = check_shared_stages(dl, L) if fs else np.zeros(d, np.uint16)
    acts = dl.acts.download(np.uint16, k * f)
    assert_ffn_close(acts, ref["acts"], "acts")
    y = dl.y.download(np.uint16, d)
    # phase 2 against the oracle fed with the device's own acts, weights and h1 (one rounding),
    # then the whole layer with the reference's relative metric
    blobs = [dl.pool_blobs()[int(c)] for c in dl.resolved.download(np.uint32, k)]
    assert_ffn_close(y, O.moe_phase2(blobs, L.oracle_offsets(), acts, dl.out_w.download(np.uint16, k), h1, d, f,
                                     bits=bits, meta=meta), "y from the device's acts")
    assert_rel_close(y, ref["y"], "y end to end")
    # The whole layer element by element against the benchmark's own bound, |y - oracle| <= 2e-3 + 1e-3 |oracle|.
    # y is an fp16 sum of fp16-rounded stages (the shared expert's output h1, the activations): where the device's
    # fp32 sum for such a stage lands on the other side of an fp16 rounding boundary, that stage moves by one fp16
    # step of ITS magnitude, and an element of y whose terms cancel inherits the step whole. So single elements
    # leave the bound; what is recorded and bounded is how many, and that none is further than two fp16 steps of
    # the vector's largest magnitude from the oracle.
    a64, b64 = f16(y).astype(np.float64), f16(ref["y"]).astype(np.float64)
    diff = np.abs(a64 - b64)
    outside = int(np.sum(diff > 2e-3 + 1e-3 * np.abs(b64)))
    step = 2.0 ** (np.floor(np.log2(np.max(np.abs(b64)))) - 10)
    print(f"\n[layer tolerance] {name}: worst |y - oracle| = {np.max(diff):.3e} = {np.max(diff) / step:.2f} fp16 steps at "
          f"max |y| = {np.max(np.abs(b64)):.2f}; {outside} of {d} elements outside 2e-3 + 1e-3|b|")
    assert np.max(diff) <= LAYER_WORST_STEPS * step and outside <= LAYER_OUTSIDE_SHARE * d, (np.max(diff), step, outside)
    assert np.array_equal(dl.hidden.download(np.uint16, d), O.residual_add_f16(L.hidden.copy(), y))

    # the operators called one after another give the same bytes as the fused entry point
    y_fused, acts_fused = y.copy(), dl.acts.download(np.uint16, k * f)
    dl.hidden.upload(L.hidden)
    dl.moe.encode_router(dl.router_w, dl.router_s, dl.router_b, dl.x, dl.eff_scale, dl.expert_scale,
                         dl.logit_bias, dl.out_idx, dl.out_w, ne, d, k)
    dl.moe.encode_residency_classification(dl.out_idx, dl.pool.table, dl.hit_count, dl.hit_pos, dl.miss_count,
                                           dl.miss_pos, dl.miss_exp, dl.resolved, k, ne)
    residual = dl.h1
    if fs:
        dl.moe.encode_shared_expert(dl.shared["gate"], dl.shared["up"], dl.shared["down"], L.shared_bits, dl.x,
                                    dl.shared_scratch, dl.h1, d, fs)
    else:
        dl.h1.fill(0)
    dl.moe.encode_spec_phase1(dl.pool, dl.resolved, dl.off, dl.x, dl.acts, d, f, k)
    dl.moe.encode_spec_phase2(dl.pool, dl.resolved, dl.off, dl.acts, dl.out_w, residual, dl.y, dl.hidden, d, f, k)
    assert np.array_equal(dl.acts.download(np.uint16, k * f), acts_fused)
    assert np.array_equal(dl.y.download(np.uint16, d), y_fused)


def _swept_layer_configs():
    """Forty configurations of the fused layer drawn once from a fixed seed: 4 to 256 experts, 1 to 8 positions, sizes any
    multiple of 64 up to 2,048, the three router widths, with and without a shared expert, both code widths and both
    metadata types."""
    rng = np.random.default_rng(0x5EED7A7E)
    out = []
    for i in range(40):
        d, f = (int(64 * rng.integers(1, 33)) for _ in range(2))
        ne = int(rng.choice([4, 8, 16, 24, 32, 40, 64, 100, 128, 160, 256]))
        k = int(rng.integers(1, min(ne, 8) + 1))
        bits, meta = int(rng.choice([4, 8])), int(rng.choice([S.META_BF16, S.META_F16]))
        rbits, fs = int(rng.choice([0, 4, 8])), int(rng.choice([0, 64, 256, 512, 1024]))
        if d * f * ne > 150_000_000:  # keep the synthetic pool small: the routes then go over eight experts
            ne = max(k, 8)
        out.append((f"sweep-{i}-d{d}-f{f}-e{ne}-k{k}", d, f, ne, k, bits, meta, rbits, fs))
    return out


@pytest.mark.parametrize("cfg", _swept_layer_configs(), ids=[c[0] for c in _swept_layer_configs()])
def test_decode_layer_config_sweep(gpu, cfg):
    test_decode_layer_matches_oracle_and_split_calls(gpu, cfg)


@pytest.mark.parametrize("ne,k,same", [(32, 4, 32), (64, 8, 64), (64, 8, 5), (256, 8, 256), (256, 8, 11), (40, 8, 40)])
def test_decode_layer_ties_go_to_the_lower_index(gpu, ne, k, same):
    """The fused layer's own select (every phase-1 wave and the workgroup that writes the lists select from the route table:
    one entry a lane up to 64 experts, four sorted entries a lane above): `same` identical router rows give `same` equal
    keys, and equal keys must come out in index order wherever they rank."""
    L = Layer(0x71E5 + ne + same, 128, 64, ne, k)
    L.router_w[:same] = L.router_w[0]
    dl = DeviceLayer(gpu, L)
    dl.moe.encode_decode_layer(dl.layer_args())
    ref = oracle_layer(L, dl)
    idx = dl.out_idx.download(np.uint32, k)
    assert np.array_equal(idx, ref["indices"]), (idx, ref["indices"])
    tied = [int(i) for i in idx if i < same]
    assert tied == list(range(len(tied))), tied  # the lowest indices of the tied group, in order
    assert np.array_equal(dl.resolved.download(np.uint32, k), ref["classify"]["resolved_slots"])
    # the waves of phase 1 selected the same experts: their activations are the oracle's
    assert_ffn_close(dl.acts.download(np.uint16, k * 64), ref["acts"], "acts")


def test_decode_layer_is_deterministic(gpu):
    L = Layer(0x5EED0002, 2048, 512, 256, 8, shared_f=512)
    dl = DeviceLayer(gpu, L)
    outs = []
    for _ in range(3):
        dl.hidden.upload(L.hidden)
        dl.moe.encode_decode_layer(dl.layer_args())
        outs.append((dl.y.download(np.uint16, 2048), dl.hidden.download(np.uint16, 2048),
                     dl.out_idx.download(np.uint32, 8)))
    for o in outs[1:]:
        assert all(np.array_equal(a, b) for a, b in zip(o, outs[0]))


def test_decode_layer_one_launch_at_a_time(gpu):
    """The layer's three launches encoded one by one (with other work on the stream between them) give the bytes
    of the one call; a mask outside 1...7 is refused."""
    L = Layer(0x5EED0002, 2048, 512, 64, 8, shared_f=512)
    dl = DeviceLayer(gpu, L)
    dl.moe.encode_decode_layer(dl.layer_args())
    want = (dl.y.download(np.uint16, 2048), dl.hidden.download(np.uint16, 2048), dl.out_idx.download(np.uint32, 8),
            dl.acts.download(np.uint16, 8 * 512))
    dl.hidden.upload(L.hidden)
    for b in (dl.y, dl.out_idx, dl.acts):
        b.fill(0x5A)
    other = gpu.empty(4096)
    for launches in (1, 2, 4):
        dl.moe.encode_decode_layer_launches(dl.layer_args(), launches)
        other.fill(launches)  # unrelated work on the same stream
    got = (dl.y.download(np.uint16, 2048), dl.hidden.download(np.uint16, 2048), dl.out_idx.download(np.uint32, 8),
           dl.acts.download(np.uint16, 8 * 512))
    assert all(np.array_equal(a, b) for a, b in zip(got, want))
    for bad in (0, 8):
        with pytest.raises(capi.ShrikeError, match="mask"):
            dl.moe.encode_decode_layer_launches(dl.layer_args(), bad)


def test_multi_chunk_pool_addressing(gpu):
    """The same cells through a pool split into several chunks (ExpertCellArena chunking)."""
    d, f, k, ne = 256, 128, 4, 12
    L = Layer(21, d, f, ne, k)
    one = DeviceLayer(gpu, L)
    padded = (L.stride + capi.POOL_PAGE - 1) // capi.POOL_PAGE * capi.POOL_PAGE
    many = DeviceLayer(gpu, L, chunk_bytes=5 * padded + 100)  # 5 cells per chunk -> 3 chunks
    assert many.pool.bases.contents.cells_per_chunk == 5
    outs = []
    for dl in (one, many):
        dl.moe.encode_decode_layer(dl.layer_args())
        outs.append(dl.y.download(np.uint16, d))
    assert np.array_equal(outs[0], outs[1])


def test_argument_errors_are_reported_not_trapped(gpu):
    moe = gpu.MoE(128, 64, 16, 8)
    with pytest.raises(capi.ShrikeError, match="topK"):
        moe.encode_router(gpu.empty(16), None, None, gpu.empty(16), gpu.empty(16), gpu.empty(16), gpu.empty(16),
                          gpu.empty(64), gpu.empty(32), 16, 128, 9)
    with pytest.raises(capi.ShrikeError, match="multiple"):
        moe.encode_router(gpu.empty(16), None, None, gpu.empty(16), gpu.empty(16), gpu.empty(16), gpu.empty(16),
                          gpu.empty(64), gpu.empty(32), 16, 100, 8)
    with pytest.raises(capi.ShrikeError):
        gpu.MoE(128, 64, 16, 9)
    with pytest.raises(capi.ShrikeError):
        gpu.ExpertPool(0, 4096, 4)


@pytest.mark.parametrize("d,f,ne,k,t,bits", [(2880, 2880, 6, 4, 4, 4), (2880, 2880, 5, 4, 3, 8), (2304, 1024, 24, 8, 16, 8), (512, 256, 16, 4, 7, 4),
                                            (2880, 2880, 32, 4, 4, 4), (2880, 2880, 32, 4, 4, 8)])  # the last two: config 4 as it is stated
def test_batched_decode_operators_equal_the_single_token_ones(gpu, d, f, ne, k, t, bits):
    """A batch of independent decode tokens (config 4: 4 tokens; config 5: 16 sequences): resolve,
    phase 1 and phase 2 with the token dimension on the grid give, per token, the bytes of the
    single-token operators, which the tests above hold to the oracle; routes come from the
    block router and are checked against the oracle bit for bit."""
    L = Layer(0x5EED0004, d, f, ne, k, bits=bits)
    resident = [e for e in range(ne) if e % 5 != 3]  # some experts miss
    dl = DeviceLayer(gpu, L, resident=resident)
    stride = d + 16
    x = S.activations_f16(L.tree, "batch.x", t * stride)
    hidden0 = S.activations_f16(L.tree, "batch.hidden", t * d)
    dx = gpu.dev(x)
    pf = gpu.Prefill(dl.moe)
    idx, w = gpu.empty(4 * t * k), gpu.empty(2 * t * k)
    pf.encode_block(dl.router_w, dl.router_s, dl.router_b, dx, dl.eff_scale, dl.expert_scale, dl.logit_bias, idx, w,
                    gpu.empty(pf.router_workspace_bytes(t, ne, d)), t, ne, d, k, stride)
    resolved, misses = gpu.empty(4 * t * k), gpu.empty(4)
    dl.moe.encode_resolve_batch(idx, dl.pool.table, resolved, t * k, ne, misses)
    acts = gpu.empty(2 * t * k * f)
    dl.moe.encode_phase1_batch(dl.pool, resolved, dl.off, dx, stride, acts, d, f, k, t)
    residual = gpu.dev(S.activations_f16(L.tree, "batch.residual", t * d))
    y, hid = gpu.empty(2 * t * d), gpu.dev(hidden0)
    dl.moe.encode_phase2_batch(dl.pool, resolved, dl.off, acts, w, residual, y, hid, d, f, k, t)
    gpu.synchronize()
    h_idx, h_w = idx.download(np.uint32, t * k), w.download(np.uint16, t * k)
    ref_idx, _, _ = O.prefill_router(L.router_dict(), x, t, d, k, stride=stride)
    assert np.array_equal(h_idx, ref_idx)
    h_res = resolved.download(np.uint32, t * k)
    want = [dl.cell_of.get(int(e), SENT) for e in h_idx]
    assert h_res.tolist() == want
    assert int(misses.download(np.uint32, 1)[0]) == sum(1 for c in want if c == SENT)
    all_acts, all_y, all_hid = acts.download(np.uint16, t * k * f), y.download(np.uint16, t * d), hid.download(np.uint16, t * d)
    res_host = residual.download(np.uint16, t * d)
    for tok in range(t):
        one_x = gpu.dev(np.ascontiguousarray(x[tok * stride:tok * stride + d]))
        one_res = gpu.dev(h_res[tok * k:(tok + 1) * k].copy())
        dl.moe.encode_spec_phase1(dl.pool, one_res, dl.off, one_x, dl.acts, d, f, k)
        one_hid = gpu.dev(hidden0[tok * d:(tok + 1) * d].copy())
        dl.moe.encode_spec_phase2(dl.pool, one_res, dl.off, dl.acts, gpu.dev(h_w[tok * k:(tok + 1) * k].copy()),
                                  gpu.dev(res_host[tok * d:(tok + 1) * d].copy()), dl.y, one_hid, d, f, k)
        gpu.synchronize()
        live = np.repeat(np.array(want[tok * k:(tok + 1) * k]) != SENT, f)
        assert np.array_equal(all_acts[tok * k * f:(tok + 1) * k * f][live], dl.acts.download(np.uint16, k * f)[live])
        assert np.array_equal(all_y[tok * d:(tok + 1) * d], dl.y.download(np.uint16, d))
        assert np.array_equal(all_hid[tok * d:(tok + 1) * d], one_hid.download(np.uint16, d))
    # and against the oracle for the first token
    blobs = [None if c == SENT else dl.pool_blobs()[c] for c in want[:k]]
    off = L.oracle_offsets()
    ref_acts = O.moe_phase1(blobs, off, np.ascontiguousarray(x[:d]), d, f, bits, L.meta)
    live0 = np.repeat(np.array(want[:k]) != SENT, f)
    assert_ffn_close(all_acts[:k * f][live0], ref_acts[live0], "token 0 activations")
    ref_y = O.moe_phase2(blobs, off, np.ascontiguousarray(all_acts[:k * f]), h_w[:k].copy(), res_host[:d].copy(), d, f, bits, L.meta)
    assert_ffn_close(all_y[:d], ref_y, "token 0 y from the device's activations")


@pytest.mark.parametrize("d,f,ne,k,t,bits,router_bits", [(2880, 2880, 32, 4, 4, 4, 0), (2880, 2880, 32, 4, 4, 8, 0), (512, 256, 40, 8, 16, 4, 8),
                                                          (2304, 1024, 256, 8, 5, 8, 0), (256, 128, 8, 3, 1, 4, 4)])
def test_decode_layer_for_a_batch_equals_the_layer_token_by_token(gpu, d, f, ne, k, t, bits, router_bits):
    """shrike_hip_moe_decode_layer_batch: the three launches with the token on the grid give, for every token, the
    routes, cells, y and hidden bytes of shrike_hip_moe_decode_layer on that token alone (which the tests above hold
    to the oracle); routes also against the oracle bit for bit. Some experts are missing from the pool."""
    L = Layer(0x5EED0044 + bits, d, f, ne, k, bits=bits, router_bits=router_bits)
    L.logit_bias = S.f32_to_bf16_bits(L.tree.key("bias").normal(ne, std=0.01))
    resident = [e for e in range(ne) if e % 7 != 2]
    dl = DeviceLayer(gpu, L, resident=resident)
    stride = d + 24
    x = S.activations_f16(L.tree, "batch.x", t * stride)
    hidden0 = S.activations_f16(L.tree, "batch.hidden", t * d)
    a = dl.layer_args()
    dx, dhid, dy = gpu.dev(x), gpu.dev(hidden0), gpu.dev(np.full(t * d, 0xD4D0, np.uint16))
    idx, w, res = gpu.empty(4 * t * k).fill(0xA5), gpu.empty(2 * t * k).fill(0xA5), gpu.empty(4 * t * k).fill(0xA5)
    acts = gpu.empty(2 * t * k * f)
    a.x, a.hidden, a.y, a.out_indices, a.out_weights, a.resolved_slots, a.acts = dx.ptr, dhid.ptr, dy.ptr, idx.ptr, w.ptr, res.ptr, acts.ptr
    for name in ("hit_count", "hit_positions", "miss_count", "miss_positions", "miss_experts"):
        setattr(a, name, None)  # a batch writes no lists
    dl.moe.encode_decode_layer_batch(a, t, stride)
    gpu.synchronize()
    h_idx, h_w, h_res = idx.download(np.uint32, t * k), w.download(np.uint16, t * k), res.download(np.uint32, t * k)
    ref_idx, ref_w, _ = O.prefill_router(L.router_dict(), x, t, d, k, stride=stride)
    assert np.array_equal(h_idx, ref_idx)
    assert h_res.tolist() == [dl.cell_of.get(int(e), SENT) for e in h_idx]
    assert SENT in h_res.tolist() or t * k < 8
    all_y, all_hid = dy.download(np.uint16, t * d), dhid.download(np.uint16, t * d)
    for tok in range(t):
        b = dl.layer_args()
        one_x, one_hid = gpu.dev(np.ascontiguousarray(x[tok * stride:tok * stride + d])), gpu.dev(hidden0[tok * d:(tok + 1) * d].copy())
        b.x, b.hidden = one_x.ptr, one_hid.ptr
        dl.moe.encode_decode_layer(b)
        gpu.synchronize()
        assert np.array_equal(dl.out_idx.download(np.uint32, k), h_idx[tok * k:(tok + 1) * k])
        assert np.array_equal(dl.out_w.download(np.uint16, k), h_w[tok * k:(tok + 1) * k])
        assert np.array_equal(dl.resolved.download(np.uint32, k), h_res[tok * k:(tok + 1) * k])
        assert np.array_equal(dl.y.download(np.uint16, d), all_y[tok * d:(tok + 1) * d]), f"token {tok}: y differs from the one-token layer"
        assert np.array_equal(one_hid.download(np.uint16, d), all_hid[tok * d:(tok + 1) * d])
    # what the entry point refuses
    lib = capi.load()
    assert lib.shrike_hip_moe_decode_layer_batch(dl.moe.handle, None, C.byref(a), 17, stride) != 0 and "tokens" in capi.last_error()
    assert lib.shrike_hip_moe_decode_layer_batch(dl.moe.handle, None, C.byref(a), t, d - 8) != 0
    shared = Layer(0x5EED0045, 256, 128, 8, 2, shared_f=128)
    sdl = DeviceLayer(gpu, shared)
    assert lib.shrike_hip_moe_decode_layer_batch(sdl.moe.handle, None, C.byref(sdl.layer_args()), 2, 256) != 0
    assert "shared expert" in capi.last_error()


@pytest.mark.parametrize("bits", [4, 8])
def test_config4_stack_of_24_layers_for_four_tokens(gpu, bits):
    """Config 4 as it is stated: 4 independent tokens through 24 stacked gpt-oss-shape layers (hidden = intermediate =
    2880, 32 experts, top-4), every layer with a pool and a router of its own, the residual stream (`hidden`) carried
    from layer to layer and each layer's x a fresh seeded row block. Every layer's routes for every token equal the
    oracle's router bit for bit; three layers' y rows are held to the oracle stage by stage for two tokens; and the
    residual stream after the last layer equals the fp16 sum, layer by layer, of the y rows the device produced."""
    d = f = 2880
    ne, k, t, n_layers = 32, 4, 4, 24
    L = Layer(0x5EED0004, d, f, ne, k, bits=bits, meta=S.META_F16)
    base = DeviceLayer(gpu, L)
    routers = [S.router_f16(L.tree, f"layer.{l}.router.w", ne, d) for l in range(n_layers)]
    xs = [S.activations_f16(L.tree, f"layer.{l}.x", t * d) for l in range(n_layers)]
    hidden0 = S.activations_f16(L.tree, "stack.hidden", t * d)
    d_hidden = gpu.dev(hidden0)
    # layers share layer 0's blobs but each has a pool of its own with its own expert -> cell map
    pools, cell_of = [base.pool], [base.cell_of]
    for l in range(1, n_layers):
        pool = gpu.ExpertPool(ne, L.stride, ne)
        cells = {}
        for e in range(ne):
            cell = (e * 5 + l) % ne
            capi.check(capi.load().shrike_hip_memcpy_d2d(pool.cell_ptr(cell), base.pool.cell_ptr(base.cell_of[e]), L.stride), "d2d")
            pool.publish(e, cell, capi.RESIDENT)
            cells[e] = cell
        pools.append(pool)
        cell_of.append(cells)
    idx, w, res = gpu.empty(4 * t * k), gpu.empty(2 * t * k), gpu.empty(4 * t * k)
    acts, y = gpu.empty(2 * t * k * f), gpu.empty(2 * t * d)
    ys, routes, all_acts = [], [], []
    for l in range(n_layers):
        a = base.layer_args()
        rw, dx = gpu.dev(routers[l]), gpu.dev(xs[l])
        a.router_weights = rw.ptr
        a.pool, a.pool_slot_stride, a.residency = pools[l].bases, pools[l].stride, pools[l].table
        a.x, a.hidden, a.y, a.out_indices, a.out_weights, a.resolved_slots, a.acts = dx.ptr, d_hidden.ptr, y.ptr, idx.ptr, w.ptr, res.ptr, acts.ptr
        base.moe.encode_decode_layer_batch(a, t, d)
        gpu.synchronize()
        ys.append(y.download(np.uint16, t * d))
        routes.append((idx.download(np.uint32, t * k), w.download(np.uint16, t * k), res.download(np.uint32, t * k)))
        all_acts.append(acts.download(np.uint16, t * k * f) if l in (0, 11, 23) else None)
    off = L.oracle_offsets()
    router = L.router_dict()
    for l in range(n_layers):
        router["weights"] = routers[l]
        ref_idx, ref_w, _ = O.prefill_router(router, xs[l], t, d, k)
        got_idx, got_w, got_res = routes[l]
        assert np.array_equal(got_idx, ref_idx), f"layer {l}: routes differ from the oracle's"
        assert np.max(np.abs(f16(got_w) - f16(ref_w))) <= 1e-3
        assert got_res.tolist() == [cell_of[l][int(e)] for e in got_idx]
    for l in (0, 11, 23):
        for tok in (0, 3):
            experts = routes[l][0][tok * k:(tok + 1) * k]
            blobs = [L.blobs[int(e)] for e in experts]
            x_row = np.ascontiguousarray(xs[l][tok * d:(tok + 1) * d])
            dev_acts = np.ascontiguousarray(all_acts[l][tok * k * f:(tok + 1) * k * f])
            assert_ffn_close(dev_acts, O.moe_phase1(blobs, off, x_row, d, f, bits, L.meta), f"layer {l} token {tok}: activations")
            ref_y = O.moe_phase2(blobs, off, dev_acts, routes[l][1][tok * k:(tok + 1) * k].copy(), np.zeros(d, np.uint16), d, f, bits, L.meta)
            assert_ffn_close(ys[l][tok * d:(tok + 1) * d], ref_y, f"layer {l} token {tok}: y from the device's activations")
    want = hidden0.copy()
    for l in range(n_layers):
        want = O.residual_add_f16(want, ys[l])
    assert np.array_equal(d_hidden.download(np.uint16, t * d), want), "the residual stream after 24 layers"
    assert len({tuple(r[0].tolist()) for r in routes}) == n_layers, "every layer routes on its own"


@pytest.mark.parametrize("bits,resident_of_selection", [(4, 5), (8, 0), (4, 8)])
def test_decode_with_misses_equals_the_resident_layer(gpu, bits, resident_of_selection):
    """The speculative pass and the agreed fixup: a token whose selection is partly (or wholly) absent from a
    12-cell pool gives the bytes of the all-resident layer; the next token over the same selection hits."""
    d, f, ne, k, cells = 512, 256, 32, 8, 12
    L = Layer(0x5EED0071 + bits, d, f, ne, k, bits=bits)
    full = DeviceLayer(gpu, L)
    residual = np.zeros(d, np.uint16)  # no shared expert: the fused layer's residual is zero
    full.moe.encode_decode_layer(full.layer_args())
    want_y, want_hidden = full.y.download(np.uint16, d), full.hidden.download(np.uint16, d)
    want_idx = full.out_idx.download(np.uint32, k)
    selection = want_idx.tolist()
    others = [e for e in range(ne) if e not in selection]
    resident = selection[:resident_of_selection] + others[: cells - resident_of_selection - 2]

    small = DeviceLayer(gpu, L, cells=cells, resident=[])
    small.moe.stream = gpu.Stream()
    cache = HL.SlotCache(cells, ne)
    store = gpu.PinnedBuffer(ne * L.stride)
    for e in range(ne):
        store.array[e * L.stride:(e + 1) * L.stride] = L.blobs[e]
    warm = cache.plan(resident)
    small.pool.execute_plan(cache, warm, store, L.stride, L.stride)
    gpu.synchronize()
    layer = runners.DecodeLayerWithMisses(small.moe, small.pool, cache, small.off, store, L.stride, L.stride)
    router = dict(weights=small.router_w, eff_scale=small.eff_scale, expert_scale=small.expert_scale, bias=small.logit_bias)
    d_res = gpu.dev(residual)
    layer.run(router, small.x, d_res, small.y, small.hidden)
    small.moe.stream.synchronize()
    assert np.array_equal(layer.idx.download(np.uint32, k), want_idx)
    assert layer.fixups == (0 if resident_of_selection == k else 1)
    assert np.array_equal(small.y.download(np.uint16, d), want_y)
    assert np.array_equal(small.hidden.download(np.uint16, d), want_hidden)
    st = cache.statistics(L.stride)
    assert st.misses == len(resident) + (k - resident_of_selection) and st.loading_slots == 0
    assert all(cache.entry(e) >> 32 == capi.RESIDENT for e in selection)
    assert [small.pool.entry(e) for e in range(ne)] == [cache.entry(e) for e in range(ne)]
    # the next token over the same selection: no fixup, the same bytes
    small.hidden.upload(L.hidden)
    layer.run(router, small.x, d_res, small.y, small.hidden)
    small.moe.stream.synchronize()
    assert layer.fixups == (0 if resident_of_selection == k else 1)
    assert np.array_equal(small.y.download(np.uint16, d), want_y)
    assert np.array_equal(small.hidden.download(np.uint16, d), want_hidden)


@pytest.mark.parametrize("d,f,ne,k,fs,rbits,bits,with_delta", [
    (2048, 512, 64, 8, 512, 0, 4, True),     # the headline shape with fewer experts
    (256, 128, 16, 4, 0, 0, 4, True),        # no shared expert: the head launch carries router rows only
    (2880, 192, 32, 4, 0, 8, 8, False),      # ragged rows, affine router, no residual add
    (512, 256, 32, 8, 256, 4, 4, True),
])
def test_decode_layer_with_the_norm_fused_ahead(gpu, d, f, ne, k, fs, rbits, bits, with_delta):
    """residual_add_rmsnorm_bf16w in the head launch's prologue: x, routes, acts, y and the residual stream
    equal, bit for bit, the stand-alone norm kernel followed by the layer."""
    L = Layer(0x5EED0081 + d, d, f, ne, k, bits=bits, router_bits=rbits, shared_f=fs)
    delta = S.f32_to_f16_bits(L.tree.key("norm.delta").normal(d, std=0.5))
    weight = S.f32_to_bf16_bits(L.tree.key("norm.weight").uniform(0.5, 1.5, d))
    eps = 1e-6
    d_delta, d_weight = gpu.dev(delta), gpu.dev(weight)

    apart = DeviceLayer(gpu, L)
    gpu.residual_add_rmsnorm_bf16w(apart.hidden, d_delta if with_delta else None, d_weight, apart.x, d, eps, 1)
    apart.moe.encode_decode_layer(apart.layer_args())

    fused = DeviceLayer(gpu, L)
    fused.x.fill(0x5A)
    args = fused.layer_args()
    args.norm_delta = d_delta.ptr if with_delta else None
    args.norm_weight, args.norm_eps = d_weight.ptr, eps
    fused.moe.encode_decode_layer(args)
    gpu.synchronize()

    want_hidden = L.hidden.copy()
    want_x = O.residual_add_rmsnorm_bf16w(want_hidden, delta if with_delta else None, weight, eps)
    assert np.array_equal(fused.x.download(np.uint16, d), want_x), "the normalised row differs from the oracle's"
    for name, count, dtype in (("x", d, np.uint16), ("out_idx", k, np.uint32), ("out_w", k, np.uint16),
                               ("acts", k * f, np.uint16), ("y", d, np.uint16), ("hidden", d, np.uint16)):
        assert np.array_equal(getattr(fused, name).download(dtype, count), getattr(apart, name).download(dtype, count)), name
    y = fused.y.download(np.uint16, d)
    assert np.array_equal(fused.hidden.download(np.uint16, d), O.residual_add_f16(want_hidden, y))
    # a second call on the same buffers is a second step of the residual stream, not a repeat of the first
    fused.moe.encode_decode_layer(args)
    gpu.residual_add_rmsnorm_bf16w(apart.hidden, d_delta if with_delta else None, d_weight, apart.x, d, eps, 1)
    apart.moe.encode_decode_layer(apart.layer_args())
    assert np.array_equal(fused.hidden.download(np.uint16, d), apart.hidden.download(np.uint16, d))


# ------------------------------------------------- family epilogues on the decode kernels

FAMILY = [  # d, f, k, bits, act, additive
    (2880, 2880, 4, 4, capi.ACT_CLAMPED_SWIGLU, True),    # gpt-oss: additive biases + clamped SwiGLU (moe.metal:257-288)
    (2880, 2880, 4, 8, capi.ACT_CLAMPED_SWIGLU, True),
    (704, 192, 8, 4, capi.ACT_CLAMPED_SWIGLU, True),
    (2048, 512, 8, 4, capi.ACT_GELU_TANH, False),         # GELU-tanh (moe.metal:98-105)
    (2048, 512, 8, 8, capi.ACT_GELU_TANH, False),
    (192, 320, 3, 8, capi.ACT_GELU_TANH, True),
    (704, 192, 8, 4, capi.ACT_SILU, True),                # the biases without the clamp
]


@pytest.mark.parametrize("d,f,k,bits,act,additive", FAMILY)
def test_decode_family_epilogues_against_oracle(gpu, d, f, k, bits, act, additive):
    """Phase 1 and phase 2 of the decode kernels with the gpt-oss epilogue (additive expert biases ahead of
    the GLU and behind the down projection, clamped SwiGLU) and with GELU-tanh, each stage against the oracle."""
    L = Layer(0x5EED0F00 + d + bits + 8 * act, d, f, k, k, bits=bits, additive_biases=additive)
    dl = DeviceLayer(gpu, L, moe_kwargs=dict(activation=act, additive_biases=additive))
    resolved = np.array([dl.cell_of[e] for e in range(k)], np.uint32)
    d_res = gpu.dev(resolved)
    dl.moe.encode_spec_phase1(dl.pool, d_res, dl.off, dl.x, dl.acts, d, f, k)
    acts = dl.acts.download(np.uint16, k * f)
    blobs = [dl.pool_blobs()[int(s)] for s in resolved]
    ref_acts = O.moe_phase1(blobs, L.oracle_offsets(), L.x, d, f, bits=bits, meta=L.meta, act=act, additive_biases=additive)
    assert_ffn_close(acts, ref_acts, "phase-1 acts")
    if additive:  # the biases matter at this tolerance: without them the oracle is far away
        plain = O.moe_phase1(blobs, L.oracle_offsets(), L.x, d, f, bits=bits, meta=L.meta, act=act, additive_biases=False)
        assert np.max(np.abs(f16(plain) - f16(ref_acts))) > 2e-2
    w = S.f32_to_f16_bits(L.tree.key("w").uniform(0.05, 0.3, k))
    residual = S.activations_f16(L.tree, "residual", d)
    hidden = L.hidden.copy()
    dl.acts.upload(ref_acts)
    dl.moe.encode_spec_phase2(dl.pool, d_res, dl.off, dl.acts, gpu.dev(w), gpu.dev(residual), dl.y, dl.hidden, d, f, k)
    ref_y = O.moe_phase2(blobs, L.oracle_offsets(), ref_acts, w, residual, d, f, bits=bits, meta=L.meta,
                         additive_biases=additive, hidden_f16=hidden)
    y = dl.y.download(np.uint16, d)
    assert_ffn_close(y, ref_y, "phase-2 y")
    if additive:
        plain_y = O.moe_phase2(blobs, L.oracle_offsets(), ref_acts, w, residual, d, f, bits=bits, meta=L.meta, additive_biases=False)
        assert np.max(np.abs(f16(plain_y) - f16(ref_y))) > 2e-2
    assert np.array_equal(dl.hidden.download(np.uint16, d), O.residual_add_f16(L.hidden.copy(), y))


def test_gpt_oss_layer_with_its_epilogue_matches_the_oracle(gpu):
    """The fused layer entry with gpt-oss's family switches at its shape: routes bit for bit, y against the oracle."""
    d, f, ne, k = 2880, 2880, 32, 4
    L = Layer(0x5EED0F44, d, f, ne, k, bits=4, additive_biases=True)
    dl = DeviceLayer(gpu, L, moe_kwargs=dict(activation=capi.ACT_CLAMPED_SWIGLU, additive_biases=True))
    dl.moe.encode_decode_layer(dl.layer_args())
    ref = oracle_layer(L, dl, act=O.ACT_CLAMPED_SWIGLU)
    assert np.array_equal(dl.out_idx.download(np.uint32, k), ref["indices"])
    acts = dl.acts.download(np.uint16, k * f)
    assert_ffn_close(acts, ref["acts"], "acts")
    blobs = [dl.pool_blobs()[int(c)] for c in dl.resolved.download(np.uint32, k)]
    y = dl.y.download(np.uint16, d)
    assert_ffn_close(y, O.moe_phase2(blobs, L.oracle_offsets(), acts, dl.out_w.download(np.uint16, k), np.zeros(d, np.uint16),
                                     d, f, bits=4, meta=L.meta, additive_biases=True), "y from the device's acts")
    assert_rel_close(y, ref["y"], "y end to end")


# ----------------------------------------------------------------------- the router pair

@pytest.mark.parametrize("ne,d,k,rbits,sigmoid", [(256, 2048, 8, 8, False), (256, 2048, 8, 0, False), (32, 2880, 4, 4, False),
                                                  (256, 2304, 8, 8, True)])
def test_router_pair_equals_two_single_routers(gpu, ne, d, k, rbits, sigmoid):
    """MoE.encodeRouterPair: this layer's router and the next layer's over the same row in one launch; both halves'
    logits, indices and weights are those of two single-router calls, bit for bit."""
    first = Layer(0x5EED0AA0 + rbits, d, 64, ne, k, router_bits=rbits, label="layer.7")
    second = Layer(0x5EED0AB0 + rbits, d, 64, ne, k, router_bits=rbits, label="layer.8")
    for L, seed in ((first, "a"), (second, "b")):
        L.logit_bias = S.f32_to_bf16_bits(L.tree.key("bias" + seed).normal(ne, std=0.01))
        L.eff_scale = S.f32_to_bf16_bits(L.tree.key("eff" + seed).uniform(0.5, 1.5, d))
    kw = dict(sigmoid=True, scaling=2.446) if sigmoid else {}
    a = DeviceLayer(gpu, first, resident=[], moe_kwargs=kw)
    b = DeviceLayer(gpu, second, resident=[], moe_kwargs=kw)
    escale = a.expert_scale
    singles = []
    for dl in (a, b):
        dl.moe.encode_router(dl.router_w, dl.router_s, dl.router_b, a.x, dl.eff_scale, escale, dl.logit_bias,
                             dl.out_idx, dl.out_w, ne, d, k)
        singles.append((dl.moe.logits(ne).copy(), dl.out_idx.download(np.uint32, k), dl.out_w.download(np.uint16, k)))
    assert not np.array_equal(singles[0][1], singles[1][1]), "the fixture's two routers must differ"
    outs = [(gpu.empty(4 * k).fill(0xFF), gpu.empty(2 * k).fill(0xFF)) for _ in range(2)]
    ops = [dict(weights=dl.router_w, scales=dl.router_s, biases=dl.router_b, effective_scale=dl.eff_scale,
                logit_bias=dl.logit_bias, out_indices=o[0], out_weights=o[1]) for dl, o in zip((a, b), outs)]
    probe = gpu.empty(4 * ne)
    for second_logits in (None, probe):
        a.moe.encode_router_pair(ops[0], ops[1], a.x, escale, ne, d, k, second_logits=second_logits)
        got_first = a.moe.logits(ne)
        got_second = a.moe.pair_logits(ne) if second_logits is None else probe.download(np.float32, ne)
        assert np.array_equal(got_first.view(np.uint32), singles[0][0].view(np.uint32))
        assert np.array_equal(got_second.view(np.uint32), singles[1][0].view(np.uint32))
        for o, want in zip(outs, singles):
            assert np.array_equal(o[0].download(np.uint32, k), want[1])
            assert np.array_equal(o[1].download(np.uint16, k), want[2])
    # and the first half against the oracle
    ref_logits = O.router_logits(first.router_w, first.router_s, first.router_b, rbits, first.x, first.eff_scale, ne, d)
    assert np.array_equal(singles[0][0].view(np.uint32), ref_logits.view(np.uint32))
    if not sigmoid:
        ref_idx, _ = O.router_select(ref_logits, first.expert_scale, first.logit_bias, k)
        assert np.array_equal(singles[0][1], ref_idx)
