"""GPU parity of the prefill operators behind the C ABI: the router for a token block, the
device grouping, the grouped expert FFN on the matrix cores, the token-major reduce and the
residual add. Indices, permutations, tables and the reduce are compared bit for bit; FFN
partial rows within max-abs 2e-3 / relative 1e-3 (|a-b| <= 2e-3 + 1e-3*|b|)."""
import numpy as np
import pytest

from oracle import host_logic as H
from oracle import oracle as O
from shrike_amd import capi
from shrike_amd import host as HL
from shrike_amd import synth as S
from harness import runners
from tests.helpers import Layer, assert_ffn_close, assert_rel_close, f16
from tests.test_decode_gpu import DeviceLayer

pytestmark = pytest.mark.gpu
SENT = 0xFFFFFFFF


def token_rows(L: Layer, t: int, stride: int, label="prefill.x"):
    """fp16[T, stride] activations; the tail of each row past d is filler that must not be read."""
    x = S.activations_f16(L.tree, label, t * stride).reshape(t, stride).copy()
    x[:, L.d:] = 0x7E00  # NaN: any use shows
    return x.reshape(-1)


def run_router(gpu, dl, L, hidden, t, stride):
    pf = gpu.Prefill(dl.moe)
    idx, w = gpu.empty(4 * t * L.k), gpu.empty(2 * t * L.k)
    ws = gpu.empty(pf.router_workspace_bytes(t, L.ne, L.d))
    pf.encode_block(dl.router_w, dl.router_s, dl.router_b, hidden, dl.eff_scale, dl.expert_scale, dl.logit_bias,
                    idx, w, ws, t, L.ne, L.d, L.k, stride)
    gpu.synchronize()
    return pf, idx, w, ws


@pytest.mark.parametrize("router_bits,ne,d,k,t,pad", [(0, 256, 2048, 8, 48, 0), (0, 256, 2048, 8, 5, 64), (8, 32, 2880, 4, 9, 8),
                                                      (4, 64, 512, 8, 33, 0), (8, 256, 2304, 8, 1, 0)])
def test_prefill_router_bit_exact_and_equal_to_decode(gpu, router_bits, ne, d, k, t, pad):
    L = Layer(0x5EED0003 + router_bits, d, 64, ne, k, router_bits=router_bits)
    L.logit_bias = S.f32_to_bf16_bits(L.tree.key("bias").normal(ne, std=0.01))
    L.expert_scale = S.f32_to_bf16_bits(L.tree.key("escale").uniform(0.6, 1.4, ne))
    dl = DeviceLayer(gpu, L, resident=[])
    stride = d + pad
    x = token_rows(L, t, stride)
    hidden = gpu.dev(x)
    pf, idx, w, ws = run_router(gpu, dl, L, hidden, t, stride)
    ref_idx, ref_w, ref_logits = O.prefill_router(L.router_dict(), x, t, d, k, stride=stride)
    logits = ws.download(np.float32, t * ne).reshape(t, ne)
    assert np.array_equal(logits.view(np.uint32), ref_logits.view(np.uint32)), "prefill logits differ in bits"
    got_idx, got_w = idx.download(np.uint32, t * k), w.download(np.uint16, t * k)
    assert np.array_equal(got_idx, ref_idx)
    assert np.max(np.abs(f16(got_w) - f16(ref_w))) <= 1e-3
    # the decode router on the same token gives the same bytes
    for tok in sorted({0, t // 2, t - 1}):
        one = gpu.dev(np.ascontiguousarray(x[tok * stride:tok * stride + d]))
        dl.moe.encode_router(dl.router_w, dl.router_s, dl.router_b, one, dl.eff_scale, dl.expert_scale, dl.logit_bias,
                             dl.out_idx, dl.out_w, ne, d, k)
        assert np.array_equal(dl.out_idx.download(np.uint32, k), got_idx[tok * k:(tok + 1) * k])
        assert np.array_equal(dl.out_w.download(np.uint16, k), got_w[tok * k:(tok + 1) * k])


@pytest.mark.parametrize("router_bits,ne,d,f,k,t,pad,bits", [
    (0, 64, 2048, 512, 8, 70, 0, 4),     # the fp16 logits kernel with four packed rows a wave forms the sums itself
    (0, 24, 2880, 384, 4, 21, 8, 8),     # the instance for longer rows; an odd token count, padded rows
    (0, 16, 192, 320, 3, 50, 24, 4),     # a row shorter than one wave load
    (8, 32, 512, 256, 4, 40, 0, 4),      # an affine router: the sums come from the pass of their own
    (0, 16, 512, 128, 2, 3, 0, 4)])      # a handful of tokens: the decode router's kernel, and the pass of their own
def test_router_with_group_sums_feeds_the_presummed_ffn(gpu, router_bits, ne, d, f, k, t, pad, bits):
    """shrike_hip_prefill_router_with_group_sums + shrike_hip_prefill_grouped_ffn_presummed against the two calls that
    each read `hidden` for themselves: the same logits, routes and weights, the same group sums at the head of the FFN's
    workspace, and the same partial rows, all bit for bit."""
    L = Layer(0x5EED0610 + router_bits + t, d, f, ne, k, bits=bits, router_bits=router_bits)
    L.logit_bias = S.f32_to_bf16_bits(L.tree.key("bias").normal(ne, std=0.01))
    dl = DeviceLayer(gpu, L)
    stride = d + pad
    x = token_rows(L, t, stride)
    hidden = gpu.dev(x)
    pf, idx, w, logits = run_router(gpu, dl, L, hidden, t, stride)
    routes = gpu.GroupedRoutesDevice(t * k, ne)
    pf.group_pairs(idx, w, t, k, ne, routes, residency=dl.pool.table)
    ws_bytes = pf.ffn_workspace_bytes(t, routes.max_row_tiles)
    ws, ws2 = gpu.empty(ws_bytes).fill(0xA5), gpu.empty(ws_bytes).fill(0x5A)
    partials, partials2 = (gpu.dev(np.full(t * k * d, 0xD4D0, np.uint16)) for _ in range(2))
    pf.encode_grouped_expert_gemms(dl.pool, dl.off, routes, hidden, stride, partials, ws, t, k)
    gpu.synchronize()
    # the fused pair, into buffers of its own
    idx2, w2 = gpu.empty(4 * t * k).fill(0xA5), gpu.empty(2 * t * k).fill(0xA5)
    logits2 = gpu.empty(pf.router_workspace_bytes(t, ne, d)).fill(0xA5)
    pf.encode_block(dl.router_w, dl.router_s, dl.router_b, hidden, dl.eff_scale, dl.expert_scale, dl.logit_bias,
                    idx2, w2, logits2, t, ne, d, k, stride, ffn_workspace=ws2)
    gpu.synchronize()
    assert np.array_equal(logits2.download(np.uint32, t * ne), logits.download(np.uint32, t * ne))
    assert np.array_equal(idx2.download(np.uint32, t * k), idx.download(np.uint32, t * k))
    assert np.array_equal(w2.download(np.uint16, t * k), w.download(np.uint16, t * k))
    sums = t * (d // 64)
    assert np.array_equal(ws2.download(np.uint32, sums), ws.download(np.uint32, sums)), "group sums differ from the FFN's own pass"
    pf.encode_grouped_expert_gemms(dl.pool, dl.off, routes, hidden, stride, partials2, ws2, t, k, presummed=True)
    gpu.synchronize()
    assert np.array_equal(partials2.download(np.uint16, t * k * d), partials.download(np.uint16, t * k * d))
    # what the entry point refuses
    lib = capi.load()
    assert lib.shrike_hip_prefill_router_with_group_sums(dl.moe.handle, None, dl.router_w.ptr, None, None, hidden.ptr, dl.eff_scale.ptr,
                                                         dl.expert_scale.ptr, dl.logit_bias.ptr, idx2.ptr, w2.ptr, logits2.ptr,
                                                         t, ne, d, k, stride, None) != 0
    assert "workspace" in capi.last_error()


def random_routes(seed, t, k, ne, skew=1.2):
    rng = np.random.default_rng(seed)
    p = 1.0 / np.arange(1, ne + 1) ** skew
    p = rng.permutation(p / p.sum())
    idx = np.concatenate([rng.choice(ne, size=k, replace=False, p=p) for _ in range(t)]).astype(np.uint32) if t else np.zeros(0, np.uint32)
    w = rng.integers(0, 0x3C00, size=t * k).astype(np.uint16)
    return idx, w


def expected_row_tiles(groups, cell_of):
    tiles = []
    for e, start, count in groups:
        for j in range(0, count, 64):
            tiles.append((cell_of(e), start + j, min(64, count - j), e))
    return tiles


@pytest.mark.parametrize("t,k,ne,mode", [(512, 8, 256, "plain"), (512, 8, 256, "keys"), (37, 3, 17, "plain"), (64, 4, 32, "residency"),
                                         (1, 8, 256, "plain"), (300, 2, 4, "keys"), (0, 8, 16, "plain"),
                                         (200, 1, 32, "plain"), (5000, 1, 7, "keys")])  # one expert a token: the token index is the pair index
def test_device_grouping_equals_host_grouping(gpu, t, k, ne, mode):
    idx, w = random_routes(t * 131 + k, t, k, ne)
    keys = None
    residency = None
    cell_of = lambda e: e
    if mode == "keys":
        order = np.random.default_rng(9).permutation(ne)[: max(1, ne // 2)].astype(np.uint32)
        keys = HL.expert_sort_keys(order, ne)
    if mode == "residency":
        words = np.array([H.residency_word(H.RESIDENT, 100 + e) if e % 3 else H.residency_word(H.LOADING if e % 2 else H.EMPTY, e)
                          for e in range(ne)], np.uint64)
        residency = gpu.dev(words)
        cell_of = lambda e: 100 + e if e % 3 else SENT
    routes = gpu.GroupedRoutesDevice(t * k, ne)
    pf = gpu.Prefill(gpu.MoE(64, 64, ne, min(k, 8)))
    pf.group_pairs(gpu.dev(idx) if t else None, gpu.dev(w) if t else None, t, k, ne, routes,
                   expert_sort_keys=None if keys is None else gpu.dev(keys), residency=residency)
    gpu.synchronize()
    got = routes.download()
    pairs = HL.make_token_expert_pairs(idx, w, t, k)
    host = HL.group_token_expert_pairs(pairs, t, k, ne, 16, keys)
    ref = H.group_token_expert_pairs(H.make_token_expert_pairs(idx, w, t, k), t, k, ne, 16, None if keys is None else keys.tolist())
    assert got["counts"].tolist() == ref.per_expert_counts == host.per_expert_counts.tolist()
    assert got["offsets"].tolist() == ref.per_expert_offsets == host.per_expert_offsets.tolist()
    assert [tuple(r) for r in got["sorted_pairs"].tolist()] == [p.as_tuple() for p in ref.sorted_pairs]
    assert [tuple(r) for r in got["row_tiles"].tolist()] == expected_row_tiles(ref.groups, cell_of)
    assert got["row_tile_count"] <= routes.max_row_tiles


def check_pair_stagewise(L: Layer, blob, x_row, dev_act, got_row, what, act=O.ACT_SILU):
    """Stage by stage, so that each comparison holds one rounding: the activations against the
    oracle's, the partial row against the oracle's down projection of the device's own
    activations; then the whole chain in the reference's relative-error metric."""
    off = L.oracle_offsets()
    dev_act = np.ascontiguousarray(dev_act)
    assert_ffn_close(dev_act, O.moe_phase1([blob], off, x_row, L.d, L.f, L.bits, L.meta, act, L.additive), f"{what}: activations")
    one, zero = np.array([0x3C00], np.uint16), np.zeros(L.d, np.uint16)
    assert_ffn_close(got_row, O.moe_phase2([blob], off, dev_act, one, zero, L.d, L.f, L.bits, L.meta, L.additive),
                     f"{what}: partial row from the device's activations")
    whole = O.prefill_pair_partial(blob, off, x_row, L.d, L.f, L.bits, L.meta, act, L.additive)
    assert_rel_close(got_row, whole, f"{what}: whole chain")


class WorkspaceActs:
    """The pairs' fp16 activation rows as the grouped FFN left them in its workspace: row tile j keeps rows
    [64 j, 64 j + 64), a pair sits at its place in the sorted pairs."""

    def __init__(self, routes, ws, t, d, f):
        self.tables = routes.download()
        act_off = (t * (d // 64) * 4 + 255) & ~255
        rows = routes.max_row_tiles * 64
        self.act = ws.download(np.uint16, rows * f, offset=act_off).reshape(rows, f)
        self.pos = {(int(r[0]), int(r[2])): i for i, r in enumerate(self.tables["sorted_pairs"])}

    def row(self, tok, rank):
        at = self.pos[(tok, rank)]
        for j, (cell, start, rows, expert) in enumerate(self.tables["row_tiles"].tolist()):
            if start <= at < start + rows:
                return self.act[j * 64 + at - start]
        raise AssertionError("pair not covered by a row tile")


class PrefillCase:
    def __init__(self, gpu, L: Layer, t, stride_pad=0, idx=None, moe_kwargs=None, resident=None):
        self.gpu, self.L, self.t = gpu, L, t
        self.dl = DeviceLayer(gpu, L, moe_kwargs=moe_kwargs, resident=resident)
        self.stride = L.d + stride_pad
        self.x = token_rows(L, t, self.stride)
        self.hidden = gpu.dev(self.x)
        self.pf = gpu.Prefill(self.dl.moe)
        if idx is None:
            idx, w = random_routes(t + L.ne, t, L.k, L.ne)
        else:
            w = np.random.default_rng(1).integers(0x3000, 0x3C00, size=t * L.k).astype(np.uint16)
        self.idx, self.w = idx, w
        self.routes = gpu.GroupedRoutesDevice(t * L.k, L.ne)
        self.d_idx, self.d_w = gpu.dev(idx), gpu.dev(w)
        self.pf.group_pairs(self.d_idx, self.d_w, t, L.k, L.ne, self.routes, residency=self.dl.pool.table)
        self.partials = gpu.dev(np.full(t * L.k * L.d, 0xD4D0, np.uint16))  # -77: rows nobody writes keep it
        self.ws = gpu.empty(self.pf.ffn_workspace_bytes(t, self.routes.max_row_tiles))

    def run(self):
        self.pf.encode_grouped_expert_gemms(self.dl.pool, self.dl.off, self.routes, self.hidden, self.stride, self.partials,
                                            self.ws, self.t, self.L.k)
        self.gpu.synchronize()
        return self.partials.download(np.uint16, self.t * self.L.k * self.L.d).reshape(self.t, self.L.k, self.L.d)

    def device_act(self, tok, rank):
        if not hasattr(self, "_acts"):
            self._acts = WorkspaceActs(self.routes, self.ws, self.t, self.L.d, self.L.f)
        return self._acts.row(tok, rank)

    def check_pair(self, got, tok, rank, what, act=O.ACT_SILU):
        L = self.L
        x = np.ascontiguousarray(self.x[tok * self.stride:tok * self.stride + L.d])
        check_pair_stagewise(L, L.blobs[int(self.idx[tok * L.k + rank])], x, self.device_act(tok, rank), got[tok, rank], what, act)


FFN_CASES = [
    # name, d, f, experts, k, tokens, bits, meta, stride pad
    ("small-int4", 512, 256, 16, 4, 40, 4, S.META_BF16, 0),
    ("small-int8-f16meta", 512, 256, 16, 4, 40, 8, S.META_F16, 8),
    ("q-shape-int4-f16meta", 2048, 512, 24, 8, 20, 4, S.META_F16, 0),
    ("q-shape-int8", 2048, 512, 12, 4, 12, 8, S.META_BF16, 0),
    ("long-experts-two-tiles", 256, 128, 3, 2, 110, 4, S.META_BF16, 0),
    ("ragged-k-192x320", 192, 320, 8, 3, 50, 4, S.META_F16, 0),
    ("kimi-shape-int8", 2304, 1024, 8, 2, 6, 8, S.META_BF16, 0),
]


@pytest.mark.parametrize("case", FFN_CASES, ids=[c[0] for c in FFN_CASES])
def test_grouped_ffn_against_oracle(gpu, case):
    name, d, f, ne, k, t, bits, meta, pad = case
    L = Layer(0x5EED0003, d, f, ne, k, bits=bits, meta=meta)
    pc = PrefillCase(gpu, L, t, stride_pad=pad)
    got = pc.run()
    rng = np.random.default_rng(4)
    sample = [(int(a), int(b)) for a, b in zip(rng.integers(0, t, 40), rng.integers(0, k, 40))] if t * k > 48 else \
        [(a, b) for a in range(t) for b in range(k)]
    for tok, rank in sample:
        pc.check_pair(got, tok, rank, f"{name} token {tok} rank {rank}")
    assert not np.any(np.all(got == 0xD4D0, axis=-1)), "a pair's partial row was left unwritten"


def _swept_ffn_cases():
    """Sixty chunks drawn once from a fixed seed: hidden and intermediate sizes any multiple of 64 up to 1,536 (column blocks
    that end inside a workgroup's 128 or 256 columns, k that ends inside a staged chunk of 256, group counts that are not
    multiples of four), 1 to 150 tokens over 2 to 20 experts (row tiles of one row, of 32, of 33, of 64 and more)."""
    rng = np.random.default_rng(0x5EEDFF)
    out = []
    for i in range(60):
        d, f = (int(64 * rng.integers(1, 25)) for _ in range(2))
        ne = int(rng.integers(2, 21))
        k = int(rng.integers(1, min(ne, 8) + 1))
        out.append((f"sweep-{i}-d{d}-f{f}", d, f, ne, k, int(rng.integers(1, 151)), int(rng.choice([4, 8])),
                    int(rng.choice([S.META_BF16, S.META_F16])), int(rng.choice([0, 8, 24]))))
    return out


@pytest.mark.parametrize("case", _swept_ffn_cases(), ids=[c[0] for c in _swept_ffn_cases()])
def test_grouped_ffn_shape_sweep(gpu, case):
    name, d, f, ne, k, t, bits, meta, pad = case
    L = Layer(0x5EED0300 + d + f, d, f, ne, k, bits=bits, meta=meta)
    pc = PrefillCase(gpu, L, t, stride_pad=pad)
    got = pc.run()
    rng = np.random.default_rng(5)
    sample = [(int(a), int(b)) for a, b in zip(rng.integers(0, t, 24), rng.integers(0, k, 24))] if t * k > 24 else \
        [(a, b) for a in range(t) for b in range(k)]
    for tok, rank in sample:
        pc.check_pair(got, tok, rank, f"{name} token {tok} rank {rank}")
    assert not np.any(np.all(got == 0xD4D0, axis=-1)), "a pair's partial row was left unwritten"


def test_grouped_ffn_gpt_oss_epilogues(gpu):
    # additive biases + clamped SwiGLU at the gpt-oss shape (moe.metal:257-288), 45 groups per row
    d = f = 2880
    L = Layer(0x5EED0004, d, f, 3, 2, bits=4, additive_biases=True)
    pc = PrefillCase(gpu, L, 5, moe_kwargs=dict(activation=capi.ACT_CLAMPED_SWIGLU, additive_biases=True))
    got = pc.run()
    for tok in range(5):
        for rank in range(2):
            pc.check_pair(got, tok, rank, f"gpt-oss token {tok} rank {rank}", O.ACT_CLAMPED_SWIGLU)


@pytest.mark.parametrize("d,f,ne,k,t,bits", [(512, 256, 6, 2, 70, 4), (320, 192, 5, 3, 21, 8)])
def test_grouped_ffn_gelu_tanh(gpu, d, f, ne, k, t, bits):
    # the GELU-tanh GLU of moe.metal:98-105 through the grouped kernels (prefill.metal:318-363): one- and two-tile
    # row tiles, both code widths
    L = Layer(0x5EED0009, d, f, ne, k, bits=bits, meta=S.META_F16)
    pc = PrefillCase(gpu, L, t, moe_kwargs=dict(activation=capi.ACT_GELU_TANH))
    got = pc.run()
    rng = np.random.default_rng(8)
    for tok, rank in {(int(a), int(b)) for a, b in zip(rng.integers(0, t, 30), rng.integers(0, k, 30))}:
        pc.check_pair(got, tok, rank, f"gelu token {tok} rank {rank}", O.ACT_GELU_TANH)
    # and it is not the SiLU result: the activation switch reached the kernel
    silu = PrefillCase(gpu, L, t).run()
    assert not np.array_equal(silu, got)


def test_grouped_ffn_skips_absent_experts(gpu):
    L = Layer(0x5EED0005, 256, 128, 8, 2, bits=4)
    pc = PrefillCase(gpu, L, 30, resident=[0, 1, 2, 4, 5, 7])
    got = pc.run()
    for tok in range(30):
        for rank in range(2):
            e = int(pc.idx[tok * 2 + rank])
            if e in (3, 6):
                assert np.all(got[tok, rank] == 0xD4D0)
            elif tok % 5 == 0:
                pc.check_pair(got, tok, rank, f"token {tok} rank {rank}")
            else:
                assert not np.all(got[tok, rank] == 0xD4D0)


def test_one_pair_expert_leaves_other_rows_alone(gpu):
    # PrefillGroupedRoutedMoETests+Execution.swift:657-763: a single 1-pair expert; the padded
    # rows of its tile must not leave the staging block
    L = Layer(0x5EED0006, 512, 512, 8, 1, bits=4)
    pc = PrefillCase(gpu, L, 1, idx=np.array([5], np.uint32))
    guard = pc.gpu.dev(np.full(64 * 512, 0xD4D0, np.uint16))
    got = pc.run()
    pc.check_pair(got, 0, 0, "single pair")
    assert np.all(guard.download(np.uint16, 64 * 512) == 0xD4D0)


@pytest.mark.parametrize("bits,tile_experts", [(4, 3), (8, 16), (4, 1)])
def test_streamed_batched_over_pair_ranges_equals_the_whole_chunk(gpu, bits, tile_experts):
    """encodeStreamedBatched: the chunk's routed tiles (pair ranges of groupTokenExpertPairs' tiles) one call
    each, against a residency table that holds the tile's experts only, give the partial rows of the one-pass
    grouped FFN byte for byte, each call writing its own pairs' rows and no others; then a range cut through
    an expert's rows."""
    d, f, ne, k, t = 256, 128, 12, 3, 90
    L = Layer(0x5EED0007 + bits, d, f, ne, k, bits=bits)
    whole = PrefillCase(gpu, L, t)
    want = whole.run()
    pc = PrefillCase(gpu, L, t)
    pairs = H.make_token_expert_pairs(pc.idx, pc.w, t, k)
    grouped = H.group_token_expert_pairs(pairs, t, k, ne, tile_expert_count=tile_experts)
    order = {(p.token, p.rank): i for i, p in enumerate(grouped.sorted_pairs)}
    cells = pc.dl.cell_of
    written = np.zeros((t, k), bool)
    for group_start, group_count, pair_start, pair_count in grouped.tiles:
        live = [g[0] for g in grouped.groups[group_start:group_start + group_count]]
        table = np.full(ne, capi.EMPTY << 32 | 0xFFFFFFFF, np.uint64)
        for e in live:
            table[e] = capi.RESIDENT << 32 | cells[e]
        batches = pc.pf.encode_streamed_batched(pc.dl.pool, pc.dl.off, pc.routes, pc.hidden, pc.stride, pc.partials, pc.ws,
                                                t, k, pair_start, pair_count, residency=gpu.dev(table))
        assert batches == -(-pair_count // 32)  # PrefillGroupedRoutedMoE.swift:864-921: microbatches of 32 pairs
        gpu.synchronize()
        got = pc.partials.download(np.uint16, t * k * d).reshape(t, k, d)
        for (tok, rank), at in order.items():
            if pair_start <= at < pair_start + pair_count:
                written[tok, rank] = True
        assert np.array_equal(got[written], want[written]), "a tile's rows differ from the one-pass result"
        assert np.all(got[~written] == 0xD4D0), "a call wrote rows of pairs outside its range"
    assert written.all()
    # a range that starts and ends inside experts' rows, against the grouping's own cells
    cut = PrefillCase(gpu, L, t)
    lo, count = 17, 101
    assert cut.pf.encode_streamed_batched(cut.dl.pool, cut.dl.off, cut.routes, cut.hidden, cut.stride, cut.partials, cut.ws,
                                          t, k, lo, count, pair_microbatch_rows=8) == 13
    gpu.synchronize()
    got = cut.partials.download(np.uint16, t * k * d).reshape(t, k, d)
    inside = np.zeros((t, k), bool)
    for (tok, rank), at in order.items():
        inside[tok, rank] = lo <= at < lo + count
    assert np.array_equal(got[inside], want[inside]) and np.all(got[~inside] == 0xD4D0)
    # nothing to do is not an error; a range past the chunk is
    assert cut.pf.encode_streamed_batched(cut.dl.pool, cut.dl.off, cut.routes, cut.hidden, cut.stride, cut.partials, cut.ws,
                                          t, k, 5, 0) == 0
    with pytest.raises(capi.ShrikeError):
        cut.pf.encode_streamed_batched(cut.dl.pool, cut.dl.off, cut.routes, cut.hidden, cut.stride, cut.partials, cut.ws,
                                       t, k, t * k - 3, 4)


def test_reduce_and_residual_bit_exact(gpu):
    rng = np.random.default_rng(12)
    for t, k, d in ((7, 8, 2048), (33, 4, 2880), (1, 1, 64)):
        partials = S.f32_to_f16_bits(rng.standard_normal(t * k * d).astype(np.float32))
        weights = S.f32_to_f16_bits(rng.random(t * k).astype(np.float32))
        pf = gpu.Prefill(gpu.MoE(64, 64, 8, 1))
        h2 = gpu.empty(2 * t * d)
        pf.encode_reduce_token_major(gpu.dev(partials), gpu.dev(weights), h2, t, k, d)
        gpu.synchronize()
        ref = O.prefill_reduce(partials, weights, t, k, d)
        assert np.array_equal(h2.download(np.uint16, t * d), ref)
        hidden = S.f32_to_f16_bits(rng.standard_normal(t * d).astype(np.float32))
        dh = gpu.dev(hidden)
        pf.residual_add(dh, h2, t * d)
        gpu.synchronize()
        assert np.array_equal(dh.download(np.uint16, t * d), O.residual_add_f16(hidden.copy(), ref))


def test_prefill_layer_at_full_size_agrees_with_the_decode_kernels(gpu):
    """T = 512 tokens, 256 experts, top 8 at the 35B-A3B int4 shape with the Zipf(1.1) skew: the routes of all
    512 tokens equal the oracle's router bit for bit (logits, indices), the grouping is a permutation with the
    host function's tables, 24 sampled pairs' activation and partial rows are held to the oracle stage by stage,
    the reduced rows equal the oracle's reduce of the device's partial rows, and sampled tokens' h2 agree with
    the decode kernels' y for that token alone (no shared expert, residual 0)."""
    d, f, ne, k, t = 2048, 512, 256, 8, 512
    L = Layer(0x5EED0003, d, f, ne, k, bits=4, meta=S.META_F16)
    # Zipf skew through the logit bias operand, over a seeded permutation
    perm = np.argsort(L.tree.key("zipf.perm").next(ne))
    bias = np.zeros(ne, np.float32)
    bias[perm] = -1.1 * np.log(np.arange(ne) + 1.0)
    L.logit_bias = S.f32_to_bf16_bits(bias)
    dl = DeviceLayer(gpu, L)
    x = token_rows(L, t, d)
    hidden = gpu.dev(x)
    pf, idx, w, ws = run_router(gpu, dl, L, hidden, t, d)
    routes = gpu.GroupedRoutesDevice(t * k, ne)
    pf.group_pairs(idx, w, t, k, ne, routes, residency=dl.pool.table)
    partials = gpu.dev(np.full(t * k * d, 0xD4D0, np.uint16))
    work = gpu.empty(pf.ffn_workspace_bytes(t, routes.max_row_tiles))
    pf.encode_grouped_expert_gemms(dl.pool, dl.off, routes, hidden, d, partials, work, t, k)
    h2 = gpu.empty(2 * t * d)
    pf.encode_reduce_token_major(partials, w, h2, t, k, d)
    gpu.synchronize()
    h_idx, h_w = idx.download(np.uint32, t * k), w.download(np.uint16, t * k)
    # every token's routes against the oracle's router, bit for bit
    ref_idx, ref_w, ref_logits = O.prefill_router(L.router_dict(), x, t, d, k)
    assert np.array_equal(ws.download(np.float32, t * ne).view(np.uint32), ref_logits.reshape(-1).view(np.uint32))
    assert np.array_equal(h_idx, ref_idx), "a token's routing indices differ from the oracle's"
    assert np.max(np.abs(f16(h_w) - f16(ref_w))) <= 1e-3
    counts = np.bincount(h_idx, minlength=ne)
    assert counts.max() > 64 and np.count_nonzero(counts) < ne, "the skew should give long experts and leave some without a pair"
    got = routes.download()
    host = HL.group_token_expert_pairs(HL.make_token_expert_pairs(h_idx, h_w, t, k), t, k, ne)
    assert got["counts"].tolist() == host.per_expert_counts.tolist() and int(got["counts"].sum()) == t * k
    assert got["offsets"].tolist() == host.per_expert_offsets.tolist()
    assert np.array_equal(got["sorted_pairs"], host.sorted_pairs.view(np.uint32).reshape(-1, 4))
    out = h2.download(np.uint16, t * d).reshape(t, d)
    rows = partials.download(np.uint16, t * k * d).reshape(t, k, d)
    assert not np.any(np.all(rows.reshape(t * k, d) == 0xD4D0, axis=-1))
    # sampled pairs against the oracle, stage by stage: pairs of the longest expert (two MFMA row tiles, several row
    # tiles), of an expert with a single pair if the routes have one, and 20 drawn over the chunk
    acts = WorkspaceActs(routes, work, t, d, f)
    rng = np.random.default_rng(6)
    sample = {(int(a), int(b)) for a, b in zip(rng.integers(0, t, 20), rng.integers(0, k, 20))}
    by_expert = {}
    for i, e in enumerate(h_idx.tolist()):
        by_expert.setdefault(e, []).append((i // k, i % k))
    longest = by_expert[int(np.argmax(counts))]
    sample.update([longest[0], longest[len(longest) // 2], longest[-1]])
    sample.add(by_expert[min(by_expert, key=lambda e: len(by_expert[e]))][0])
    for tok, rank in sorted(sample):
        check_pair_stagewise(L, L.blobs[int(h_idx[tok * k + rank])], np.ascontiguousarray(x[tok * d:(tok + 1) * d]),
                             acts.row(tok, rank), rows[tok, rank], f"full-size chunk token {tok} rank {rank}")
    assert np.array_equal(out.reshape(-1), O.prefill_reduce(rows.reshape(-1), h_w, t, k, d)), "reduce differs from the oracle's"
    zero = gpu.dev(np.zeros(d, np.uint16))
    for tok in (0, 1, 77, 255, 256, 511):
        one = gpu.dev(np.ascontiguousarray(x[tok * d:(tok + 1) * d]))
        dl.moe.encode_router(dl.router_w, None, None, one, dl.eff_scale, dl.expert_scale, dl.logit_bias, dl.out_idx, dl.out_w, ne, d, k)
        assert np.array_equal(dl.out_idx.download(np.uint32, k), h_idx[tok * k:(tok + 1) * k])
        cells = np.array([dl.cell_of[int(e)] for e in h_idx[tok * k:(tok + 1) * k]], np.uint32)
        dl.moe.encode_spec_phase1(dl.pool, gpu.dev(cells), dl.off, one, dl.acts, d, f, k)
        hid = gpu.dev(np.zeros(d, np.uint16))
        dl.moe.encode_spec_phase2(dl.pool, gpu.dev(cells), dl.off, dl.acts, dl.out_w, zero, dl.y, hid, d, f, k)
        gpu.synchronize()
        # The decode kernel rounds the fp32 sum over the experts once; prefill rounds each of the
        # eight partial rows to fp16 first (as the reference does), so single elements of a
        # cancelling sum move by a few fp16 steps of the largest partial: compared in the
        # reference's relative-error metric.
        assert_rel_close(out[tok], dl.y.download(np.uint16, d), f"token {tok}: prefill h2 vs decode y", tol=2e-3)


@pytest.mark.parametrize("d,fs,bits,t,gated", [(2048, 512, 4, 20, False), (2048, 512, 4, 70, True), (2304, 1024, 8, 16, True),
                                              (192, 320, 4, 70, False), (128, 64, 8, 1, True)])
def test_shared_expert_for_a_token_block(gpu, d, fs, bits, t, gated):
    """The chunk's shared expert with ONE SCALAR GATE A TOKEN (RealForwardRunner.swift:4438-4456): the gate row's
    GEMV for every token (moe.metal:1154-1193) bit for bit against the oracle, then h1[t] = shared(x_t) * sigmoid(gate[t])
    against the oracle token by token; the two-launch form (ungated block, then sigmoid_scalar_mul_rows) gives the same."""
    L = Layer(0x5EED0007, d, 64, 4, 2, bits=bits, shared_f=fs, shared_bits=bits)
    dl = DeviceLayer(gpu, L, resident=[])
    pf = gpu.Prefill(dl.moe)
    stride = d + 8
    x = token_rows(L, t, stride)
    dx = gpu.dev(x)
    h1 = gpu.dev(np.full(t * d, 0xD4D0, np.uint16))
    gates = None
    d_gates = None
    if gated:
        gate_row = S.affine_matrix(L.tree.key("shared.scalar_gate"), 1, d, 8, L.meta)
        d_gates = gpu.empty(2 * t).fill(0xFF)
        pf.encode_scalar_gate_rows(tuple(gpu.dev(a) for a in gate_row), dx, stride, d_gates, t, d)
        gates = d_gates.download(np.uint16, t)
        want_gates = O.shared_scalar_gate_rows(gate_row, x, t, d, x_stride=stride, meta=L.meta)
        assert np.array_equal(gates, want_gates), "the per-row gate differs from the oracle in bits"
        assert t == 1 or len(set(gates.tolist())) > 1
    pf.encode_shared_expert(dl.shared["gate"], dl.shared["up"], dl.shared["down"], bits, dx, stride, h1, t, fs,
                            scalar_gate=d_gates)
    gpu.synchronize()
    got = h1.download(np.uint16, t * d).reshape(t, d)
    for tok in range(t):
        xt = np.ascontiguousarray(x[tok * stride:tok * stride + d])
        gate_bits = gates[tok:tok + 1].copy() if gated else None
        ref = O.shared_expert(L.shared["gate"], L.shared["up"], L.shared["down"], xt, d, fs, bits=bits, meta=L.meta,
                              scalar_gate_f16=gate_bits)
        # gate/up -> fp16 -> act -> fp16 -> down -> fp16 (-> gate -> fp16): whole chain, the reference's metric
        assert_rel_close(got[tok], ref, f"token {tok}", tol=2e-3 if gated else 1e-3)
        # and equal to the single-token operator on the same token
        if tok in (0, t - 1):
            one = gpu.empty(2 * d)
            dl.moe.encode_shared_expert(dl.shared["gate"], dl.shared["up"], dl.shared["down"], bits, gpu.dev(xt), dl.shared_scratch,
                                        one, d, fs, scalar_gate=gpu.dev(gate_bits) if gated else None)
            gpu.synchronize()
            assert_rel_close(got[tok], one.download(np.uint16, d), f"token {tok} vs the decode operator", tol=2e-3 if gated else 1e-3)
    if gated:
        # the reference's two kernels: the ungated block, then y[t, :] *= sigmoid(gate[t]) in place
        plain = gpu.dev(np.full(t * d, 0xD4D0, np.uint16))
        pf.encode_shared_expert(dl.shared["gate"], dl.shared["up"], dl.shared["down"], bits, dx, stride, plain, t, fs)
        ungated = plain.download(np.uint16, t * d)
        pf.encode_sigmoid_scalar_mul_rows(plain, d_gates, d, t)
        gpu.synchronize()
        assert np.array_equal(plain.download(np.uint16, t * d).reshape(t, d), got), "fused and two-launch gating differ"
        # the elementwise kernel against the oracle: the device's exp may differ from libm's in the last bit
        assert_ffn_close(plain.download(np.uint16, t * d), O.sigmoid_scalar_mul_rows(ungated.copy(), gates, d, t), "sigmoid rows")


@pytest.mark.parametrize("d,f,ne,k,t,bits,slots,slru", [
    (256, 128, 48, 4, 12, 8, 16, None), (256, 128, 48, 4, 12, 4, 8, 0.5),
    (2304, 1024, 256, 8, 16, 8, 64, None),  # config 5 as it is stated: Kimi-Linear shape, 16 sequences, 64 of 256 cells
])
def test_batched_decode_through_a_pool_smaller_than_the_expert_set(gpu, d, f, ne, k, t, bits, slots, slru):
    """Config 5: several sequences, one token each, through a pool smaller than the expert set; the experts
    stream from pinned host memory in passes. Routes are bit-exact, every partial row matches the
    oracle stage by stage, the statistics (and so the miss rate) equal the slot-cache restatement's over the
    same plans, and a second step hits the cache."""
    L = Layer(0x5EED0005, d, f, ne, k, bits=bits)
    dl = DeviceLayer(gpu, L, cells=slots, resident=[])
    dl.moe.stream = gpu.Stream()
    cache = HL.SlotCache(slots, ne, slru_share=slru)
    store = gpu.PinnedBuffer(ne * L.stride)
    for e in range(ne):
        store.array[e * L.stride:(e + 1) * L.stride] = L.blobs[e]
    layer = runners.BatchedDecodeLayer(dl.moe, dl.pool, cache, dl.off, store, L.stride, L.stride, t)
    x = token_rows(L, t, d)
    hidden = gpu.dev(x)
    router = dict(weights=dl.router_w, eff_scale=dl.eff_scale, expert_scale=dl.expert_scale, bias=dl.logit_bias)
    h2 = layer.run(router, hidden, t, d)
    dl.moe.stream.synchronize()
    ref_idx, ref_w, _ = O.prefill_router(L.router_dict(), x, t, d, k)
    idx, w = layer.idx.download(np.uint32, t * k), layer.w.download(np.uint16, t * k)
    assert np.array_equal(idx, ref_idx)
    used = len(set(idx.tolist()))
    assert layer.passes == -(-used // slots) and layer.passes >= 2
    partials = layer.partials.download(np.uint16, t * k * d).reshape(t, k, d)
    # every pair stage by stage (the passes share one grouping, so a pair's activation row stays where the pass that
    # served its expert left it)
    acts = WorkspaceActs(layer.routes, layer.ffn_ws, t, d, f)
    for tok in range(t):
        xt = np.ascontiguousarray(x[tok * d:(tok + 1) * d])
        for rank in range(k):
            check_pair_stagewise(L, L.blobs[int(idx[tok * k + rank])], xt, acts.row(tok, rank), partials[tok, rank],
                                 f"token {tok} rank {rank}")
    assert np.array_equal(h2.download(np.uint16, t * d), O.prefill_reduce(partials.reshape(-1), w, t, k, d))
    st = cache.statistics(L.stride)
    assert (st.plans, st.requested_experts, st.misses, st.hits) == (layer.passes, used, used, 0)
    assert st.bytes_read == used * L.stride and st.loading_slots == 0 and st.resident_slots == min(slots, used)
    # every device residency word equals the cache's own
    assert [dl.pool.entry(e) for e in range(ne)] == [cache.entry(e) for e in range(ne)]
    # a second step over the same tokens: the experts of the last pass are still resident
    before = cache.statistics().hits
    layer.run(router, hidden, t, d)
    dl.moe.stream.synchronize()
    assert cache.statistics().hits > before
    # the miss rate over both steps is the slot-cache restatement's over the same plans
    twin = H.SlotCache(slots, ne, slru_share=slru)
    for batch in layer.plan_log:
        twin.load(batch)
    st, ts = cache.statistics(L.stride), twin.stats
    assert (st.plans, st.requested_experts, st.hits, st.misses, st.evictions, st.reloads) == tuple(
        ts[n] for n in ("plans", "requested", "hits", "misses", "evictions", "reloads"))
    assert [cache.entry(e) for e in range(ne)] == list(twin.words)
    miss_rate = st.misses / st.requested_experts
    print(f"\n[config 5] d={d} f={f} E={ne} K={k} tokens={t} cells={slots}: {used} distinct experts a step, "
          f"{layer.passes} passes, miss rate over two steps {miss_rate:.3f}")
    assert 0.0 < miss_rate < 1.0
    again = layer.partials.download(np.uint16, t * k * d)
    assert np.array_equal(again, partials.reshape(-1))  # same bytes whatever cell an expert landed in


@pytest.mark.parametrize("d,rows", [(2048, 1), (2304, 1), (2880, 3), (64, 5), (4096, 2), (2048, 512)])
def test_residual_add_rmsnorm_bit_exact(gpu, d, rows):
    """The producer of the path's input (rmsnorm.metal:96-130) against the oracle: the updated hidden rows
    and the normalised rows bit for bit, with and without the residual add."""
    tree = S.SeedTree(0x5EED0052)
    eps = 1e-6
    hidden = S.activations_f16(tree, "hidden", rows * d)
    delta = S.f32_to_f16_bits(tree.key("delta").normal(rows * d, std=0.5))
    weight = S.f32_to_bf16_bits(tree.key("weight").uniform(0.5, 1.5, d))
    for with_delta in (True, False):
        d_hidden, d_delta, d_weight, d_out = gpu.dev(hidden), gpu.dev(delta), gpu.dev(weight), gpu.empty(2 * rows * d)
        gpu.residual_add_rmsnorm_bf16w(d_hidden, d_delta if with_delta else None, d_weight, d_out, d, eps, rows)
        got_hidden, got_out = d_hidden.download(np.uint16, rows * d), d_out.download(np.uint16, rows * d)
        for r in range(rows if rows <= 8 else 4):
            h = hidden[r * d:(r + 1) * d].copy()
            want = O.residual_add_rmsnorm_bf16w(h, delta[r * d:(r + 1) * d] if with_delta else None, weight, eps)
            assert np.array_equal(got_hidden[r * d:(r + 1) * d], h)
            assert np.array_equal(got_out[r * d:(r + 1) * d], want), f"row {r} of d={d}"
    for bad_d in (20, 8192):  # not a multiple of 8; past the kernels' hidden-size ceiling
        with pytest.raises(capi.ShrikeError, match="multiple of 8"):
            gpu.residual_add_rmsnorm_bf16w(d_hidden, None, d_weight, d_out, bad_d, eps)
