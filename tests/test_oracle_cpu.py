"""The arithmetic oracle (oracle/shrike_oracle.c) against what pins it without a GPU: the
reference's own C kernel compiled in place (oracle/_ref, when it was built), the reference
tests' known answers, closed forms, and fp64 / brute-force restatements written here from the
format's definition rather than from the oracle's code."""
import math
import os

import numpy as np
import pytest

from oracle import host_logic as H
from oracle import oracle as O
from shrike_amd import synth as S


def f16(bits):
    return np.asarray(bits, np.uint16).view(np.float16).astype(np.float32)


# ------------------------------------------------------------------------------ conversions

def test_conversions_exhaustive_against_numpy():
    L = O.lib()
    for h in range(0, 65536, 1):
        v = np.uint16(h).view(np.float16)
        got = L.orc_f16_to_f32(h)
        if np.isnan(v):
            assert math.isnan(got)
        else:
            assert got == float(v)
    rng = np.random.default_rng(1)
    xs = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 10.0 ** rng.integers(-8, 6, 20000),
                         np.array([0.0, -0.0, 65504.0, 65520.0, 65519.99, 5.96e-8, 2.98e-8, 2.9802325e-8, 1e-10,
                                   np.inf, -np.inf], np.float32)]).astype(np.float32)
    with np.errstate(over="ignore"):
        want16 = xs.astype(np.float16).view(np.uint16)
    for x, w16 in zip(xs, want16):
        assert L.orc_f32_to_f16(float(x)) == int(w16), x
    # bf16: round to nearest even on the upper 16 bits (Quantization.swift:17-28)
    for x in xs:
        u = int(np.float32(x).view(np.uint32))
        want = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF
        assert L.orc_f32_to_bf16(float(x)) == want
        assert L.orc_bf16_to_f32(want) == float(np.uint32(want << 16).view(np.float32))


# ---------------------------------------------------------------------------- blob layout

def test_offsets_known_answers():  # CPUExpertFFNTests.swift:56-67, ExpertCacheBudgetTests.swift:16-18
    o, stride = O.expert_offsets(2048, 512, 4)
    assert stride == 1_769_472
    assert (o.gate_w, o.gate_s, o.up_w, o.down_w) == (0, 524_288, 589_824, 1_179_648)
    t = o.as_tuple()[:9]
    assert list(t) == sorted(t)
    assert O.expert_offsets(2048, 512, 8)[1] == 3_342_336
    assert O.expert_offsets(2880, 2880, 4)[1] == 13_996_800
    assert O.expert_offsets(2880, 2880, 8)[1] == 26_438_400
    assert O.expert_offsets(2880, 2880, 8, additive_biases=True)[1] == 26_438_400 + 17_280
    assert O.expert_offsets(2304, 1024, 8)[1] == 7_520_256
    so, sstride = S.expert_offsets(2048, 512, 4)
    assert sstride == stride and tuple(so[n] for n, _ in O.Offsets._fields_) == o.as_tuple()


# --------------------------------------------------------------------------- affine GEMV

def brute_gemv(w, s, b, x, rows, n, bits, meta):
    """w = q * scale + bias per element, in fp64, from the format's definition."""
    out = np.zeros(rows, np.float64)
    w, s, b = (np.ascontiguousarray(a).reshape(-1) for a in (w, s, b))
    sf, bf = S.meta_to_f32(s, meta).astype(np.float64), S.meta_to_f32(b, meta).astype(np.float64)
    for r in range(rows):
        row = w[r * n * bits // 8:(r + 1) * n * bits // 8]
        q = np.stack([row & 0xF, row >> 4], axis=1).reshape(-1) if bits == 4 else row
        g = np.arange(n) // 64
        out[r] = np.sum((q.astype(np.float64) * sf[r * (n // 64) + g] + bf[r * (n // 64) + g]) * x.astype(np.float64))
    return out


@pytest.mark.parametrize("rows,n", [(128, 64), (64, 512), (32, 2880)])
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("meta", [S.META_BF16, S.META_F16])
def test_gemv_against_brute_force(rows, n, bits, meta):
    rng = S.SeedTree(0x5EED0001).key(f"gemv.{rows}.{n}.{bits}.{meta}")
    w, s, b = S.affine_matrix(rng, rows, n, bits, meta)
    x = rng.normal(n).astype(np.float32)
    ref = brute_gemv(w, s, b, x, rows, n, bits, meta)
    got = O.affine_gemv(w, s, b, x, rows, n, bits, meta)
    got64 = O.affine_gemv_f64(w, s, b, x, rows, n, bits, meta)
    scale = np.abs(ref).max()
    assert np.abs(got64 - ref).max() <= 1e-9 * scale
    assert np.abs(got - ref).max() <= 1e-5 * scale  # DequantInt4GEMVReferenceTests.swift:32-53
    if bits == 4:
        assert np.array_equal(O.int4_affine_gemv(w, s, b, x, rows, n, meta), got)


@pytest.mark.skipif(O.ref_lib_path() is None, reason="oracle/_ref was not built (no reference checkout at build time)")
@pytest.mark.parametrize("rows,n", [(2048, 512), (512, 2048), (128, 64), (2880, 2880), (1024, 2304)])
def test_int4_gemv_bit_equal_to_the_reference_c(rows, n):
    rng = S.SeedTree(0x5EED0001).key(f"ref.{rows}.{n}")
    w, s, b = S.affine_matrix(rng, rows, n, 4, S.META_BF16)
    x = rng.normal(n).astype(np.float32)
    ours = O.int4_affine_gemv(w, s, b, x, rows, n, S.META_BF16)
    theirs = O.ref_int4_affine_gemv(w, s, b, x, rows, n)
    assert ours.view(np.uint32).tolist() == theirs.view(np.uint32).tolist()


def test_nibble_layout_low_even_high_odd():  # QuantizationTests.swift:36-50
    row = (np.arange(64, dtype=np.float32) - 31.5)[None, :]
    w, s, b = (a.reshape(-1) for a in S.quantize_affine(row, 4))
    lo, hi = int(w[0] & 0xF), int(w[0] >> 4)
    sc, bi = float(S.bf16_bits_to_f32(s)[0]), float(S.bf16_bits_to_f32(b)[0])
    assert abs(lo * sc + bi - row[0, 0]) <= sc + 1e-3 and abs(hi * sc + bi - row[0, 1]) <= sc + 1e-3
    e = np.zeros(64, np.float32)
    e[1] = 1.0  # picks element 1: the high nibble of byte 0
    assert abs(O.affine_gemv(w, s, b, e, 1, 64, 4)[0] - (hi * sc + bi)) < 1e-6


def test_quantiser_round_trip_bound():  # QuantizationTests.swift:8-34
    rng = S.SeedTree(0x51A71001).key("int4-affine-round-trip")
    row = rng.uniform(-1.0, 1.0, 256).astype(np.float32)[None, :]
    w, s, b = (a.reshape(-1) for a in S.quantize_affine(row, 4))
    q = np.stack([w & 0xF, w >> 4], axis=1).reshape(-1).astype(np.float32)
    rec = q * np.repeat(S.bf16_bits_to_f32(s), 64) + np.repeat(S.bf16_bits_to_f32(b), 64)
    for g in range(4):
        seg = slice(64 * g, 64 * g + 64)
        assert np.all(np.abs(rec[seg] - row[0, seg]) <= np.abs(row[0, seg]).max() / 7.0 + 1e-3)


# --------------------------------------------------------------------------- expert FFN

def closed_form_blob(d, f, meta=S.META_BF16):
    """q = 0, scale = 0, gate bias 1/64... (MoEFusedFFNTests.swift:17-55): every weight equals its
    group's bias, so gate = D/64 * 1/64 * ... reduces to sums of ones."""
    o, stride = O.expert_offsets(d, f, 4)
    blob = np.zeros(stride, np.uint8)

    def put(off, rows, n, value):
        vals = np.full(rows * (n // 64), value, np.float32)
        blob[off:off + vals.size * 2] = S.meta_bits(vals, meta).view(np.uint8)
    put(o.gate_b, f, d, 1.0 / 64)
    put(o.up_b, f, d, 0.5 / 64)
    put(o.down_b, d, f, 1.0 / 64)
    return blob, o


def test_ffn_closed_form():  # MoEFusedFFNTests.swift:868-900: D=128, F=64, 8 experts x 0.125 -> 2/(1+e^-2)
    d, f = 128, 64
    blob, o = closed_form_blob(d, f)
    x = S.f32_to_f16_bits(np.ones(d, np.float32))
    acts = O.moe_phase1([blob] * 8, o, x, d, f)
    # gate = 128/64 = 2, up = 1, act = silu(2) * 1
    assert np.allclose(f16(acts), 2.0 / (1.0 + math.exp(-2.0)), atol=1e-3)
    w = S.f32_to_f16_bits(np.full(8, 0.125, np.float32))
    zero = S.f32_to_f16_bits(np.zeros(d, np.float32))
    hidden = zero.copy()
    y = O.moe_phase2([blob] * 8, o, acts, w, zero, d, f, hidden_f16=hidden)
    # down = sum_f act / 64 = act
    assert np.allclose(f16(y), 2.0 / (1.0 + math.exp(-2.0)), atol=1e-2)
    assert np.array_equal(hidden, y)


def test_cpu_ffn_matches_fp64_chain_and_accumulates():  # CPUExpertFFNTests.swift:69-152
    d, f = 256, 128
    tree = S.SeedTree(0x5EED0001)
    blob = S.expert_blob(tree, "cpu.ffn", d, f, 4)
    o, _ = O.expert_offsets(d, f, 4)
    v = S.blob_views(blob, d, f, 4)
    x = tree.key("cpu.x").normal(d).astype(np.float32)
    gate = brute_gemv(*v["gate"], x, f, d, 4, S.META_BF16)
    up = brute_gemv(*v["up"], x, f, d, 4, S.META_BF16)
    act = gate / (1.0 + np.exp(-gate)) * up
    down = brute_gemv(*v["down"], act.astype(np.float32), d, f, 4, S.META_BF16)
    out = np.zeros(d, np.float32)
    O.cpu_expert_ffn_accumulate(blob, o, x, d, f, 0.75, out)
    assert np.abs(out - 0.75 * down).max() <= 2e-4 * max(1.0, np.abs(down).max())
    once = out.copy()
    O.cpu_expert_ffn_accumulate(blob, o, x, d, f, 0.75, out)
    assert np.allclose(out, 2 * once, rtol=1e-6, atol=1e-6)


def test_glu_variants():  # moe.metal:98-105, :257-288
    L = O.lib()
    g, u = 0.7, -1.3
    assert abs(L.orc_glu(g, u, O.ACT_SILU) - g / (1 + math.exp(-g)) * u) < 1e-6
    gelu = 0.5 * g * (1 + math.tanh(0.7978845608 * (g + 0.044715 * g ** 3)))
    assert abs(L.orc_glu(g, u, O.ACT_GELU_TANH) - gelu * u) < 1e-6
    # gpt-oss: gate clamped above at 7, up to [-7, 7], gate * sigmoid(1.702 gate) * (up + 1)
    for g, u in ((9.0, 9.0), (-9.0, -9.0), (0.5, 0.25)):
        gc, uc = min(g, 7.0), max(-7.0, min(7.0, u))
        want = gc / (1 + math.exp(-1.702 * gc)) * (uc + 1)
        assert abs(L.orc_glu(g, u, O.ACT_CLAMPED_SWIGLU) - want) < 1e-5 * max(1, abs(want))


# --------------------------------------------------------------------------------- router

def softmax_reference(logits, expert_scale, k):
    """RouterTopKTests.swift:594-620: sort by (score desc, index asc), exp(s - max) / sum, x scale."""
    order = sorted(range(len(logits)), key=lambda e: (-float(logits[e]), e))[:k]
    ex = [math.exp(float(logits[e]) - float(logits[order[0]])) for e in order]
    return order, [v / sum(ex) * float(expert_scale[e]) for v, e in zip(ex, order)]


def test_router_select_against_sorted_reference():
    rng = np.random.default_rng(7)
    ones = S.f32_to_bf16_bits(np.ones(256, np.float32))
    zeros = S.f32_to_bf16_bits(np.zeros(256, np.float32))
    for trial in range(50):
        n, k = int(rng.choice([32, 64, 128, 256])), int(rng.choice([1, 4, 8]))
        logits = rng.standard_normal(n).astype(np.float32)
        if trial % 5 == 0:
            logits[rng.integers(0, n, 6)] = logits[0]  # exact ties: the lower index wins
        scale = S.f32_to_bf16_bits((1 + rng.random(n)).astype(np.float32))
        idx, w = O.router_select(logits, scale, zeros[:n], k)
        order, weights = softmax_reference(logits, S.bf16_bits_to_f32(scale), k)
        assert idx.tolist() == order
        assert np.abs(f16(w) - np.array(weights)).max() < 5e-3  # RouterTopKTests.swift:43
    # additive bias shifts the selection (RouterTopKTests.swift:75-99)
    logits = np.linspace(-1, 1, 64).astype(np.float32)
    bias = np.zeros(64, np.float32)
    bias[0] = 100.0
    idx0, _ = O.router_select(logits, ones[:64], zeros[:64], 4)
    idx1, w1 = O.router_select(logits, ones[:64], S.f32_to_bf16_bits(bias), 4)
    assert 0 not in idx0.tolist() and idx1[0] == 0 and f16(w1)[0] > 0.99


def test_router_near_tie_resolves_like_the_sorted_reference():  # RouterTopKTests.swift:101-125
    d, e = 512, 64
    rng = S.SplitMix64(0x71E0F4A)
    pattern = rng.uniform(0.2, 1.0, d)
    hidden = rng.uniform(0.5, 1.5, d)
    gains = np.zeros(e, np.float32)
    gains[:7] = 1.0 - np.arange(7) * 0.05
    gains[7], gains[8] = 0.5, 0.5 * (1.0 + 1e-4)
    gains[9:] = 0.4 - np.arange(e - 9) * 0.02
    w = (gains[:, None] * pattern[None, :]).astype(np.float32)
    wq, ws, wb = S.quantize_affine(w, 8)
    x = S.f32_to_f16_bits(hidden.astype(np.float32))
    ones = S.f32_to_bf16_bits(np.ones(d, np.float32))
    logits = O.router_logits(wq, ws, wb, O.ROUTER_AFFINE8, x, ones, e, d)
    ref = brute_gemv(wq, ws, wb, f16(x), e, d, 8, S.META_BF16)
    assert np.abs(logits - ref).max() <= 1e-4 * np.abs(ref).max()
    idx, _ = O.router_select(logits, S.f32_to_bf16_bits(np.ones(e, np.float32)), S.f32_to_bf16_bits(np.zeros(e, np.float32)), 8)
    assert idx.tolist() == softmax_reference(ref.astype(np.float32), np.ones(e), 8)[0]
    assert idx.tolist()[7] == 8  # the 1e-4 gap is resolved, not tied


def test_sigmoid_router():  # RouterTopKTests.swift:343-368: select on sigmoid + bias, weigh by sigmoid, x 2.446
    rng = np.random.default_rng(11)
    n, k, scaling = 256, 8, 2.446
    logits = rng.standard_normal(n).astype(np.float32)
    corr = S.bf16_bits_to_f32(S.f32_to_bf16_bits((rng.standard_normal(n) * 0.1).astype(np.float32)))
    sig = 1 / (1 + np.exp(-logits.astype(np.float64)))
    order = sorted(range(n), key=lambda e: (-(np.float32(sig[e]) + np.float32(corr[e])), e))[:k]
    orig = [sig[e] for e in order]
    want = [v / (sum(orig) + 1e-20) * scaling for v in orig]
    idx, w = O.router_select(logits, S.f32_to_bf16_bits(np.ones(n, np.float32)), S.f32_to_bf16_bits(corr), k,
                             sigmoid=True, scaling=scaling)
    assert idx.tolist() == order
    assert np.abs(f16(w) - np.array(want)).max() < 5e-3


def test_fp16_router_logits_against_fp64():
    tree = S.SeedTree(0x5EED0002)
    e, d = 256, 2048
    w = S.router_f16(tree, "router.w", e, d)
    x = S.activations_f16(tree, "x", d)
    eff = S.f32_to_bf16_bits(np.ones(d, np.float32))
    got = O.router_logits(w, None, None, O.ROUTER_F16, x, eff, e, d)
    ref = f16(w).astype(np.float64).reshape(e, d) @ f16(x).astype(np.float64)
    assert np.abs(got - ref).max() <= 1e-5 * np.abs(ref).max() + 1e-6


# ---------------------------------------------------------------------- residency classify

def classify_with(cache: H.SlotCache, experts):
    table = np.array(cache.words, np.uint64)
    return O.classify(np.array(experts, np.uint32), table, cache.experts_per_layer)


def test_classify_follows_the_slot_cache_states():  # GPUExpertResidencyTests.swift:24-70
    c = H.SlotCache(2, 4)
    loading = c.plan([0])
    r = classify_with(c, [0, 1, 2, 3])
    assert r["hit_count"] == 0 and r["miss_positions"].tolist() == [0, 1, 2, 3]
    c.complete(loading)
    c.load([2])
    r = classify_with(c, [0, 1, 2, 3])
    assert r["hit_positions"].tolist() == [0, 2] and r["miss_positions"].tolist() == [1, 3]
    assert r["miss_experts"].tolist() == [1, 3]
    assert r["resolved_slots"][0] != H.U32_MAX and r["resolved_slots"][2] != H.U32_MAX
    assert r["resolved_slots"][1] == H.U32_MAX
    c.load([1, 3])
    r = classify_with(c, [0, 1, 2, 3])
    assert r["hit_positions"].tolist() == [1, 3] and r["miss_positions"].tolist() == [0, 2]
    assert c.words[0] >> 32 == H.EMPTY


def test_prefill_reduce_and_residual():  # PrefillMoETests.swift:8-64
    rng = np.random.default_rng(3)
    t, k, d = 5, 4, 64
    partials = S.f32_to_f16_bits(rng.standard_normal(t * k * d).astype(np.float32))
    weights = S.f32_to_f16_bits(rng.random(t * k).astype(np.float32))
    h2 = O.prefill_reduce(partials, weights, t, k, d)
    ref = np.einsum("tkd,tk->td", f16(partials).reshape(t, k, d).astype(np.float64), f16(weights).reshape(t, k).astype(np.float64))
    assert np.abs(f16(h2).reshape(t, d) - ref).max() <= 2e-3 * max(1.0, np.abs(ref).max())
    hidden = S.f32_to_f16_bits(rng.standard_normal(t * d).astype(np.float32))
    want = (f16(hidden) + f16(h2)).astype(np.float16)
    got = O.residual_add_f16(hidden.copy(), h2)
    assert np.array_equal(got.view(np.float16), want)


def test_int4_gemv_against_committed_reference_vectors():
    """tests/golden/ref_int4_gemv.json holds what the reference's C kernel returned for these seeded
    inputs (written by tests/golden/make_ref_gemv_vectors.py): the check that travels without the
    reference checkout."""
    import json
    import zlib
    from tests.golden.make_ref_gemv_vectors import inputs
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_int4_gemv.json")
    for case in json.load(open(path))["cases"]:
        rows, n = case["rows"], case["n"]
        w, s, b, x = inputs(rows, n)
        y = O.int4_affine_gemv(w, s, b, x, rows, n, S.META_BF16).view(np.uint32)
        assert [int(v) for v in y[:16]] == case["head"], (rows, n)
        assert zlib.crc32(y.tobytes()) == case["crc32"], (rows, n)


# ---------------------------------------------------------------- rmsnorm ahead of the router

def test_residual_add_rmsnorm_against_the_definition():
    """rmsnorm.metal:5-13, :96-130: hidden += delta in fp16; out = hidden * rsqrt(mean(hidden^2) + eps) * weight.
    Pinned by the closed form on a constant row, by fp64 on random rows, and by the reference's statement
    that the fused kernel equals residual_add_fp16 followed by the norm alone."""
    eps = 1e-6
    ones = S.f32_to_f16_bits(np.full(2048, 2.0, np.float32))
    w = S.f32_to_bf16_bits(np.full(2048, 0.5, np.float32))
    out = O.residual_add_rmsnorm_bf16w(ones.copy(), None, w, eps)
    assert np.all(S.f16_bits_to_f32(out) == np.float32(np.float16(2.0 / np.sqrt(4.0 + eps) * 0.5)))
    tree = S.SeedTree(0x5EED0051)
    for d in (64, 2048, 2304, 2880, 4096):
        hidden = S.activations_f16(tree, f"h.{d}", d)
        delta = S.f32_to_f16_bits(tree.key(f"d.{d}").normal(d, std=0.5))
        weight = S.f32_to_bf16_bits(tree.key(f"w.{d}").uniform(0.5, 1.5, d))
        h = hidden.copy()
        out = O.residual_add_rmsnorm_bf16w(h, delta, weight, eps)
        summed = (S.f16_bits_to_f32(hidden) + S.f16_bits_to_f32(delta)).astype(np.float16)
        assert np.array_equal(h, summed.view(np.uint16)), "the add rounds through fp16 storage"
        x = summed.astype(np.float64)
        want = x / np.sqrt(np.mean(x * x) + eps) * S.bf16_bits_to_f32(weight).astype(np.float64)
        got = S.f16_bits_to_f32(out).astype(np.float64)
        assert np.max(np.abs(got - want) / (np.abs(want) + 1e-3)) <= 1e-3  # one fp16 rounding of the result
        two_step = O.residual_add_f16(hidden.copy(), delta)
        assert np.array_equal(O.residual_add_rmsnorm_bf16w(two_step, None, weight, eps), out)
        assert np.array_equal(two_step, h)


# ------------------------------------------------------------ fp64 chains from the format's definition
#
# Everything below restates a function of the oracle in numpy fp64 from the DEFINITION of the format
# (w = q * scale + bias per element, low nibble = even element) and of the layer (which value is rounded to
# fp16 where, per the Metal sources cited), never from the oracle's own loops. A stage that rounds to fp16
# can land one fp16 step away from the fp64 chain (an fp32 sum next to a rounding boundary), so chains are
# held to a few fp16 steps of the vector's scale; each test also shows that a plausible mistake (operands
# swapped, a term dropped, the gate left out) breaks the same bound.

def dequant(w, s, b, rows, n, bits, meta):
    """[rows, n] fp64 weights from the format's definition."""
    w = np.ascontiguousarray(w).reshape(rows, n * bits // 8)
    q = np.stack([w & 0xF, w >> 4], axis=2).reshape(rows, n) if bits == 4 else w
    sf = S.meta_to_f32(np.ascontiguousarray(s).reshape(-1), meta).astype(np.float64).reshape(rows, n // 64)
    bf = S.meta_to_f32(np.ascontiguousarray(b).reshape(-1), meta).astype(np.float64).reshape(rows, n // 64)
    return q.astype(np.float64) * np.repeat(sf, 64, axis=1) + np.repeat(bf, 64, axis=1)


def h(v):
    """One fp16 rounding, back in fp64."""
    with np.errstate(over="ignore"):
        return np.asarray(v, np.float64).astype(np.float16).astype(np.float64)


def glu64(g, u, act):
    if act == O.ACT_SILU:
        return g / (1.0 + np.exp(-g)) * u
    if act == O.ACT_GELU_TANH:  # moe.metal:98-105
        return 0.5 * g * (1.0 + np.tanh(np.clip(0.7978845608028654 * (g + 0.044715 * g ** 3), -20, 20))) * u
    gc, uc = np.minimum(g, 7.0), np.clip(u, -7.0, 7.0)  # moe.metal:280-288
    return gc / (1.0 + np.exp(-1.702 * gc)) * (uc + 1.0)


def close_in_f16_steps(got_bits, want64, steps, what):
    """|got - want| <= steps * (one fp16 step at the vector's largest magnitude)."""
    got = f16(got_bits).astype(np.float64)
    scale = max(float(np.max(np.abs(want64))), 1e-3)
    step = 2.0 ** (np.floor(np.log2(scale)) - 10)
    worst = float(np.max(np.abs(got - want64)))
    return worst <= steps * step, f"{what}: worst |diff| {worst:.3e} vs {steps} fp16 steps of {step:.3e}"


def shared_chain(sh, x64, d, fs, bits, meta, act, gate_bits=None, swap=False, drop_gate=False):
    """dequant_int4.metal:177-179 (the GEMVs write half), :283-287 (act = half(glu)), :322-329 (gated tail)."""
    wg, wu, wd = (dequant(*sh[n], r, c, bits, meta) for n, r, c in (("gate", fs, d), ("up", fs, d), ("down", d, fs)))
    g, u = h(wg @ x64), h(wu @ x64)
    if swap:
        g, u = u, g
    y = h(wd @ h(glu64(g, u, act)))
    if gate_bits is not None and not drop_gate:
        y = h(y / (1.0 + np.exp(-float(f16(gate_bits)[0]))))
    return g, u, y


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("d,fs", [(256, 128), (2048, 512)])
@pytest.mark.parametrize("gated", [False, True])
def test_shared_expert_against_fp64_chain(bits, d, fs, gated):
    tree = S.SeedTree(0x5EED0A10 + bits + d)
    meta = S.META_BF16
    sh = {n: S.affine_matrix(tree.key(f"shared.{n}"), r, c, bits, meta)
          for n, r, c in (("gate", fs, d), ("up", fs, d), ("down", d, fs))}
    x = S.activations_f16(tree, "x", d)
    gate_bits = S.f32_to_f16_bits(np.array([-0.4], np.float32)) if gated else None
    g64, u64, y64 = shared_chain(sh, f16(x).astype(np.float64), d, fs, bits, meta, O.ACT_SILU, gate_bits)
    g, u = O.shared_gate_up(sh["gate"], sh["up"], x, d, fs, bits=bits, meta=meta)
    ok, msg = close_in_f16_steps(g, g64, 1, "gate rows")
    assert ok, msg
    ok, msg = close_in_f16_steps(u, u64, 1, "up rows")
    assert ok, msg
    assert not np.array_equal(g, u)
    # the down stage alone from the oracle's own gate/up: one rounding of act, one of y (and one more when gated)
    y_from = O.shared_down(sh["down"], g, u, d, fs, bits=bits, meta=meta, scalar_gate_f16=gate_bits)
    wd = dequant(*sh["down"], d, fs, bits, meta)
    y_stage = h(wd @ h(glu64(f16(g).astype(np.float64), f16(u).astype(np.float64), O.ACT_SILU)))
    if gated:
        y_stage = h(y_stage / (1.0 + np.exp(-float(f16(gate_bits)[0]))))
    ok, msg = close_in_f16_steps(y_from, y_stage, 2, "down from given gate/up")
    assert ok, msg
    # the whole chain; the composition equals its two halves
    y = O.shared_expert(sh["gate"], sh["up"], sh["down"], x, d, fs, bits=bits, meta=meta, scalar_gate_f16=gate_bits)
    assert np.array_equal(y, y_from)
    ok, msg = close_in_f16_steps(y, y64, 3, "shared expert")
    assert ok, msg
    # what the bound catches
    _, _, swapped = shared_chain(sh, f16(x).astype(np.float64), d, fs, bits, meta, O.ACT_SILU, gate_bits, swap=True)
    assert not close_in_f16_steps(y, swapped, 3, "")[0], "gate and up swapped must not pass"
    if gated:
        _, _, ungated = shared_chain(sh, f16(x).astype(np.float64), d, fs, bits, meta, O.ACT_SILU, gate_bits, drop_gate=True)
        assert not close_in_f16_steps(y, ungated, 3, "")[0], "a dropped scalar gate must not pass"


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("act", [O.ACT_SILU, O.ACT_GELU_TANH, O.ACT_CLAMPED_SWIGLU])
@pytest.mark.parametrize("additive", [False, True])
def test_routed_phases_against_fp64_chain(bits, act, additive):
    """moe.metal:261-288 (additive biases ahead of the GLU, clamped SwiGLU), :829 (acts are half), :933-939
    (partial = half weight * (down + bias); y = half(residual + sum in rank order)), :889-893 (hidden += y)."""
    d, f, k = 192, 128, 3
    meta = S.META_BF16
    tree = S.SeedTree(0x5EED0A20 + bits + 16 * act + int(additive))
    blobs = [S.expert_blob(tree, f"e{e}", d, f, bits, meta, additive) for e in range(k)]
    off, _ = O.expert_offsets(d, f, bits, additive)
    soff, _ = S.expert_offsets(d, f, bits, additive)
    x = S.activations_f16(tree, "x", d)
    x64 = f16(x).astype(np.float64)
    acts = O.moe_phase1(blobs, off, x, d, f, bits=bits, meta=meta, act=act, additive_biases=additive)
    w_bits = S.f32_to_f16_bits(np.array([0.5, 0.3, 0.2], np.float32))
    residual = S.activations_f16(tree, "residual", d)
    hidden = S.activations_f16(tree, "hidden", d)
    hidden_out = hidden.copy()
    y = O.moe_phase2(blobs, off, acts, w_bits, residual, d, f, bits=bits, meta=meta, additive_biases=additive,
                     hidden_f16=hidden_out)

    def ab(blob, name, n):
        return S.bf16_bits_to_f32(blob[soff[name]:soff[name] + 2 * n].view(np.uint16)).astype(np.float64)

    def chain(bias_after_glu=False, drop_down_bias=False):
        acc = f16(residual).astype(np.float64)
        all_acts = []
        for e in range(k):
            v = S.blob_views(blobs[e], d, f, bits, additive)
            g, u = dequant(*v["gate"], f, d, bits, meta) @ x64, dequant(*v["up"], f, d, bits, meta) @ x64
            if additive and not bias_after_glu:
                g, u = g + ab(blobs[e], "gate_ab", f), u + ab(blobs[e], "up_ab", f)
            a = glu64(g, u, act)
            if additive and bias_after_glu:
                a = a + ab(blobs[e], "gate_ab", f)
            a = h(a)
            all_acts.append(a)
            down = dequant(*v["down"], d, f, bits, meta) @ a
            if additive and not drop_down_bias:
                down = down + ab(blobs[e], "down_ab", d)
            acc = acc + float(f16(w_bits)[e]) * down
        return np.concatenate(all_acts), h(acc)

    a64, y64 = chain()
    ok, msg = close_in_f16_steps(acts, a64, 1, "acts")
    assert ok, msg
    ok, msg = close_in_f16_steps(y, y64, 2, "y")
    assert ok, msg
    assert np.array_equal(hidden_out, (f16(hidden) + f16(y)).astype(np.float16).view(np.uint16))
    if additive:
        wrong_acts, _ = chain(bias_after_glu=True)
        assert not close_in_f16_steps(acts, wrong_acts, 1, "")[0], "the bias added after the GLU must not pass"
        _, wrong_y = chain(drop_down_bias=True)
        assert not close_in_f16_steps(y, wrong_y, 2, "")[0], "a dropped down bias must not pass"
    # a sentinel position keeps its acts and adds nothing (moe.metal:986, :1037-1038)
    keep = np.full(k * f, 0x3555, np.uint16)
    part = O.moe_phase1([blobs[0], None, blobs[2]], off, x, d, f, bits=bits, meta=meta, act=act,
                        additive_biases=additive, acts=keep.copy())
    assert np.array_equal(part[f:2 * f], keep[f:2 * f]) and np.array_equal(part[:f], acts[:f])


@pytest.mark.parametrize("kind", [O.ROUTER_F16, O.ROUTER_AFFINE8, O.ROUTER_AFFINE4])
def test_router_logits_with_effective_scale_against_fp64(kind):
    """moe.metal:324-364: logit = sum (q*s + b) * (half(hidden) * bf16(effective_scale))."""
    e, d = 48, 704
    tree = S.SeedTree(0x5EED0A30 + kind)
    dense = tree.key("w").normal(e * d, std=0.02).reshape(e, d)
    x = S.activations_f16(tree, "x", d)
    eff = S.f32_to_bf16_bits(tree.key("eff").uniform(0.25, 1.75, d))
    xs = f16(x).astype(np.float64) * S.bf16_bits_to_f32(eff).astype(np.float64)
    if kind == O.ROUTER_F16:
        w = S.f32_to_f16_bits(dense.reshape(-1)).reshape(e, d)
        got = O.router_logits(w, None, None, kind, x, eff, e, d)
        ref = f16(w).astype(np.float64).reshape(e, d) @ xs
    else:
        wq, ws, wb = S.quantize_affine(dense.astype(np.float32), kind)
        got = O.router_logits(wq, ws, wb, kind, x, eff, e, d)
        ref = dequant(wq, ws, wb, e, d, kind, S.META_BF16) @ xs
    bound = 1e-5 * np.abs(ref).max() + 1e-6
    assert np.abs(got - ref).max() <= bound
    plain = (f16(w).astype(np.float64).reshape(e, d) if kind == O.ROUTER_F16
             else dequant(wq, ws, wb, e, d, kind, S.META_BF16)) @ f16(x).astype(np.float64)
    assert np.abs(got - plain).max() > 100 * bound, "ignoring the effective scale must not pass"


def test_cpu_layer_against_fp64_chain():
    """CPUExpertFFN.swift:102-140 over several experts, one task each: out += w_e * down_e(silu(gate_e x) * up_e x),
    everything in fp32 with no fp16 rounding between the stages; any thread count gives the same bits."""
    d, f, n = 256, 128, 5
    tree = S.SeedTree(0x5EED0A40)
    blobs = [S.expert_blob(tree, f"e{e}", d, f, 4) for e in range(n)]
    off, _ = O.expert_offsets(d, f, 4)
    x = tree.key("x").normal(d).astype(np.float32)
    rw = np.array([0.4, 0.25, 0.2, 0.1, 0.05], np.float32)
    want = np.zeros(d, np.float64)
    for e in range(n):
        v = S.blob_views(blobs[e], d, f, 4)
        g = dequant(*v["gate"], f, d, 4, S.META_BF16) @ x.astype(np.float64)
        u = dequant(*v["up"], f, d, 4, S.META_BF16) @ x.astype(np.float64)
        want += float(rw[e]) * (dequant(*v["down"], d, f, 4, S.META_BF16) @ (g / (1.0 + np.exp(-g)) * u))
    outs = [O.cpu_layer_fp32(blobs, rw, off, x, d, f, threads) for threads in (1, 3, 8)]
    assert np.abs(outs[0] - want).max() <= 2e-4 * max(1.0, np.abs(want).max())  # CPUExpertFFNTests.swift:69-113
    assert all(np.array_equal(o.view(np.uint32), outs[0].view(np.uint32)) for o in outs[1:])
    dropped = O.cpu_layer_fp32(blobs[:4], rw[:4], off, x, d, f, 2)
    assert np.abs(dropped - want).max() > 2e-4 * max(1.0, np.abs(want).max()), "a dropped expert must not pass"


@pytest.mark.parametrize("d", [2048, 2304, 192])
def test_per_row_scalar_gate_against_fp64(d):
    """moe.metal:1154-1207: gate[row] = half(dequant8(W) . x_row); y[row, :] = half(y[row, :] * sigmoid(gate[row]))."""
    rows, stride = 7, d + 24
    tree = S.SeedTree(0x5EED0A50 + d)
    w, s, b = S.affine_matrix(tree.key("gate.row"), 1, d, 8, S.META_BF16)
    x = S.activations_f16(tree, "x", rows * stride)
    gate = O.shared_scalar_gate_rows((w, s, b), x, rows, d, x_stride=stride)
    xm = f16(x).astype(np.float64).reshape(rows, stride)[:, :d]
    want = xm @ dequant(w, s, b, 1, d, 8, S.META_BF16)[0]
    assert np.all(np.abs(f16(gate) - want) <= 1e-3 * np.abs(want) + 1e-4), "one fp16 rounding of an fp32 sum"
    assert len(set(gate.tolist())) == rows, "every row has its own gate"
    y = S.activations_f16(tree, "y", rows * d)
    out = O.sigmoid_scalar_mul_rows(y.copy(), gate, d, rows)
    sig = 1.0 / (1.0 + np.exp(-f16(gate).astype(np.float64)))
    want_y = h(f16(y).astype(np.float64).reshape(rows, d) * sig[:, None])
    diff = np.abs(f16(out).astype(np.float64).reshape(rows, d) - want_y)
    assert np.all(diff <= np.abs(want_y) * 2.0 ** -10 + 1e-7)
    one_gate = h(f16(y).astype(np.float64).reshape(rows, d) * sig[0])
    assert np.max(np.abs(f16(out).astype(np.float64).reshape(rows, d) - one_gate)) > 1e-2, \
        "row 0's gate applied to every row must not pass"
