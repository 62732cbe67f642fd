// The reference's closed-form FFN case (MoEFusedFFNTests.swift:17-55, :868-900) through the C++ mirror of
// the operator surface on the GPU: codes 0, scales 0, gate bias 1/64, up bias 0.5/64, down bias 1/64, x = 1,
// D = 128, F = 64, eight experts of weight 0.125, residual 0 -> every output is 2 / (1 + e^-2) within 0.01.
// Decode: phase 1 + phase 2 over resolved slots. Prefill: device grouping, grouped GEMMs, token-major reduce.
// Build: g++ -std=c++17 -I include tests/cpp/gpu_harness.cpp -L shrike_amd -lshrikehip
#include <cmath>
#include <cstdio>
#include <cstring>
#include <vector>

#include "shrike.hpp"

using namespace shrike;

static int failures = 0;
#define EXPECT(cond)                                                      \
    do {                                                                  \
        if (!(cond)) {                                                    \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            ++failures;                                                   \
        }                                                                 \
    } while (0)

struct Device {  // a device allocation with host copies in and out
    void *p;
    uint64_t bytes;
    explicit Device(uint64_t n) : p(shrike_hip_malloc(n)), bytes(n) {
        if (!p) throw Error(ENOMEM, shrike_hip_last_error());
    }
    template <typename T>
    explicit Device(const std::vector<T> &host) : Device(uint64_t(host.size() * sizeof(T))) {
        check(shrike_hip_memcpy_h2d(p, host.data(), bytes));
    }
    ~Device() { shrike_hip_free(p); }
    Device(const Device &) = delete;
    template <typename T>
    std::vector<T> download() const {
        std::vector<T> out(bytes / sizeof(T));
        check(shrike_hip_memcpy_d2h(out.data(), p, bytes));
        return out;
    }
    template <typename T>
    T *as() const { return static_cast<T *>(p); }
};

static float halfToFloat(uint16_t h) {  // normal numbers and zero are all this test sees
    const int e = (h >> 10) & 31, m = h & 1023;
    const float v = e == 0 ? std::ldexp(float(m), -24) : std::ldexp(float(1024 + m), e - 25);
    return (h & 0x8000) ? -v : v;
}

int main() {
    const uint32_t d = 128, f = 64, experts = 8, k = 8;
    const uint16_t one = 0x3C00, eighth = 0x3000, half = 0x3800;           // fp16 1, 0.125, 0.5
    const uint16_t b64 = 0x2400, b128 = 0x2000;                            // fp16 1/64, 0.5/64
    const float want = 2.0f / (1.0f + std::exp(-2.0f));
    check(shrike_hip_init(0));

    shrike_expert_offsets off;
    const uint64_t stride = shrike_expert_offsets_make(d, f, 4, 0, &off);
    EXPECT(stride >= 3u * (uint64_t(f) * d / 2u + 2u * 2u * f * (d / 64u)));  // codes, scales and biases of three projections
    std::vector<uint8_t> blob(stride, 0);
    auto fill = [&](uint32_t at, uint32_t count, uint16_t bits) {
        for (uint32_t i = 0; i < count; ++i) std::memcpy(&blob[at + 2u * i], &bits, 2);
    };
    fill(off.gate_b_off, f * (d / 64), b64);
    fill(off.up_b_off, f * (d / 64), b128);
    fill(off.down_b_off, d * (f / 64), b64);

    shrike_moe_desc desc{};
    desc.d = d; desc.f = f; desc.num_experts = experts; desc.top_k = k;
    desc.routed_weight_bits = 4; desc.meta_dtype = SHRIKE_META_F16; desc.activation = SHRIKE_ACT_SILU;
    MoE moe(desc);
    ExpertPool pool(experts, stride, experts);
    for (uint32_t e = 0; e < experts; ++e) {
        pool.upload(e, blob.data(), stride, nullptr);
        pool.publish(e, e, SHRIKE_RESIDENCY_RESIDENT, nullptr);
    }
    check(shrike_hip_device_synchronize());
    EXPECT(pool.residencyEntry(3) == (uint64_t(SHRIKE_RESIDENCY_RESIDENT) << 32 | 3u));

    // ---- decode: one token over all eight experts
    {
        std::vector<uint32_t> slots(k);
        for (uint32_t i = 0; i < k; ++i) slots[i] = (i * 3u) % experts;  // any order: the experts are alike
        Device resolved(slots), x(std::vector<uint16_t>(d, one)), weights(std::vector<uint16_t>(k, eighth));
        Device residual(std::vector<uint16_t>(d, 0)), hidden(std::vector<uint16_t>(d, half));
        Device acts(uint64_t(2) * k * f), y(uint64_t(2) * d);
        moe.encodeSpecPhase1U16Load(nullptr, pool, resolved.as<uint32_t>(), off, x.p, acts.p, d, f, k);
        moe.encodeSpecPhase2Reduce(nullptr, pool, resolved.as<uint32_t>(), nullptr, off, acts.p, weights.p, residual.p, y.p, hidden.p,
                                   d, f, k);
        check(shrike_hip_device_synchronize());
        for (uint16_t v : acts.download<uint16_t>()) EXPECT(std::fabs(halfToFloat(v) - want) <= 0.01f);
        for (uint16_t v : y.download<uint16_t>()) EXPECT(std::fabs(halfToFloat(v) - want) <= 0.01f);
        for (uint16_t v : hidden.download<uint16_t>()) EXPECT(std::fabs(halfToFloat(v) - (0.5f + want)) <= 0.01f);  // hidden += y
    }

    // ---- prefill: five tokens, two experts each, through grouping, the grouped GEMMs and the reduce
    {
        const uint32_t t = 5, kk = 2;
        shrike_moe_desc pdesc = desc;
        pdesc.top_k = kk;
        MoE pmoe(pdesc);
        std::vector<uint32_t> indices(t * kk);
        for (uint32_t i = 0; i < t * kk; ++i) indices[i] = (i * 5u + i / kk) % experts;
        for (uint32_t tok = 0; tok < t; ++tok)
            if (indices[tok * kk] == indices[tok * kk + 1]) indices[tok * kk + 1] = (indices[tok * kk] + 1u) % experts;
        Device idx(indices), w(std::vector<uint16_t>(t * kk, half)), x(std::vector<uint16_t>(t * d, one));
        const uint32_t maxTiles = shrike_hip_group_max_row_tiles(t * kk, experts);
        Device sorted(uint64_t(16) * t * kk), offsets(4 * experts), counts(4 * experts), tiles(uint64_t(16) * maxTiles), tileCount(4);
        const shrike_hip_grouped_routes routes{sorted.p, offsets.as<uint32_t>(), counts.as<uint32_t>(),
                                               tiles.as<shrike_row_tile>(), tileCount.as<uint32_t>()};
        PrefillMoEGrouping::encodeGroupPairs(nullptr, idx.as<uint32_t>(), w.p, t, kk, experts, nullptr, pool.residencyTable(), routes);
        Device partials(uint64_t(2) * t * kk * d), h2(uint64_t(2) * t * d);
        Device workspace(PrefillGroupedRoutedMoE::workspaceBytes(t, maxTiles, d, f));
        PrefillGroupedRoutedMoE::encodeGroupedExpertGEMMs(pmoe, nullptr, pool, off, routes, maxTiles, x.p, d, partials.p, workspace.p,
                                                          workspace.bytes, t, d, f, kk);
        PrefillMoE::encodeReduceTokenMajor(nullptr, partials.p, w.p, h2.p, t, kk, d);
        check(shrike_hip_device_synchronize());
        const auto pairs = sorted.download<shrike_token_expert_pair>();
        for (uint32_t i = 1; i < t * kk; ++i) EXPECT(pairs[i - 1].expert <= pairs[i].expert);  // sorted by expert
        uint32_t total = 0;
        for (uint32_t c : counts.download<uint32_t>()) total += c;
        EXPECT(total == t * kk);
        for (uint16_t v : partials.download<uint16_t>()) EXPECT(std::fabs(halfToFloat(v) - want) <= 0.01f);
        for (uint16_t v : h2.download<uint16_t>()) EXPECT(std::fabs(halfToFloat(v) - want) <= 0.01f);  // 0.5 + 0.5 of the same value
        // one routed tile of the chunk through the streamed-batched entry: the first three sorted pairs
        Device again(std::vector<uint16_t>(size_t(t) * kk * d, 0xD4D0));
        const uint32_t batches = PrefillGroupedRoutedMoE::encodeStreamedBatched(pmoe, nullptr, pool, off, routes, maxTiles, pool.residencyTable(),
                                                                               0, 3, x.p, d, again.p, workspace.p, workspace.bytes, t, d, f, kk, 2);
        check(shrike_hip_device_synchronize());
        EXPECT(batches == 2);
        const auto rows = again.download<uint16_t>();
        for (uint32_t i = 0; i < t * kk; ++i) {
            const shrike_token_expert_pair &p = pairs[i];
            const uint16_t v = rows[(size_t(p.token) * kk + p.rank) * d + 7];
            if (i < 3) EXPECT(std::fabs(halfToFloat(v) - want) <= 0.01f);
            else EXPECT(v == 0xD4D0);
        }
    }
    std::printf(failures ? "%d checks failed\n" : "all gpu checks passed\n", failures);
    return failures ? 1 : 0;
}
