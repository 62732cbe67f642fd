// Host-side integer logic of the prefill routed path: pair records, the grouping
// permutation, the resident-first sweep order and the staging-wave planner.
#include <algorithm>
#include <climits>
#include <cstring>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "../../include/shrike_host.h"
#include "host_common.h"

using shrike::set_error;

namespace {

// ---- grouping ---------------------------------------------------------------------------

int grouping_fail(shrike_grouped_routes *out, int code, int64_t a, int64_t b, const char *fmt, ...) {
    if (out) {
        out->error_value[0] = a;
        out->error_value[1] = b;
    }
    char text[160];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(text, sizeof text, fmt, ap);
    va_end(ap);
    set_error("%s", text);
    return code;
}

// ---- sweep order ------------------------------------------------------------------------

struct RowsOf {
    const std::unordered_map<uint32_t, int64_t> &rows;
    int64_t operator()(uint32_t e) const {
        auto it = rows.find(e);
        return it == rows.end() ? 0 : it->second;
    }
};

std::vector<uint32_t> heaviest_first(std::vector<uint32_t> experts, const RowsOf &rows) {
    std::sort(experts.begin(), experts.end(), [&](uint32_t l, uint32_t r) {
        const int64_t lr = rows(l), rr = rows(r);
        if (lr != rr) return lr > rr;
        return l < r;
    });
    return experts;
}

// PrefillMoEGrouping.swift:234-261: heaviest first into the lightest bin with room, ties to
// the lower bin; the bins may come pre-seeded.
void pack_into(const std::vector<uint32_t> &experts, std::vector<std::vector<uint32_t>> &bins,
               const RowsOf &rows, size_t tile_width) {
    std::vector<int64_t> weights(bins.size(), 0);
    for (size_t i = 0; i < bins.size(); ++i)
        for (uint32_t e : bins[i]) weights[i] += rows(e);
    for (uint32_t e : heaviest_first(experts, rows)) {
        ptrdiff_t best = -1;
        int64_t best_weight = INT64_MAX;
        for (size_t i = 0; i < bins.size(); ++i) {
            if (bins[i].size() < tile_width && weights[i] < best_weight) {
                best_weight = weights[i];
                best = ptrdiff_t(i);
            }
        }
        if (best < 0) break;
        bins[size_t(best)].push_back(e);
        weights[size_t(best)] += rows(e);
    }
}

// PrefillMoEGrouping.swift:203-226
std::vector<uint32_t> pack_by_rows(const std::vector<uint32_t> &experts, const RowsOf &rows, size_t tile_width) {
    std::vector<uint32_t> flat;
    if (experts.empty()) return flat;
    std::vector<std::vector<uint32_t>> bins((experts.size() + tile_width - 1) / tile_width);
    pack_into(experts, bins, rows, tile_width);
    for (auto &b : bins) flat.insert(flat.end(), b.begin(), b.end());
    return flat;
}

// PrefillMoEGrouping.swift:179-190
std::vector<uint32_t> fallback_order(const std::vector<uint32_t> &resident, const std::vector<uint32_t> &absent,
                                     const RowsOf &rows, size_t tile_width) {
    const size_t tail = std::min<size_t>(96, absent.size());  // residentFirstFallbackTail
    const size_t head = absent.size() - tail;
    std::vector<uint32_t> order = pack_by_rows(resident, rows, tile_width);
    auto h = pack_by_rows(std::vector<uint32_t>(absent.begin(), absent.begin() + ptrdiff_t(head)), rows, tile_width);
    auto t = pack_by_rows(std::vector<uint32_t>(absent.begin() + ptrdiff_t(head), absent.end()), rows, tile_width);
    order.insert(order.end(), h.begin(), h.end());
    order.insert(order.end(), t.begin(), t.end());
    return order;
}

// ---- wave planner -----------------------------------------------------------------------

constexpr int64_t kBodyTile = 64;  // MPPPrefillInt4QMM.tileM
constexpr int64_t kTailTile = 32;

struct Planner {
    shrike_routed_expert_block *blocks;
    size_t block_capacity;
    shrike_routed_expert_wave *waves;
    size_t wave_capacity;
    size_t block_count = 0, wave_count = 0;
    size_t wave_first_block = 0;

    void add_block(uint32_t slot, int64_t pair_start, int64_t rows, int64_t staging_row, int64_t tile_start) {
        if (block_count < block_capacity)
            blocks[block_count] = {slot, uint32_t(pair_start), uint32_t(rows), uint32_t(staging_row), uint32_t(tile_start)};
        ++block_count;
    }
    void add_wave(int64_t padded_rows, int64_t tail_rows) {
        if (wave_count < wave_capacity)
            waves[wave_count] = {uint32_t(wave_first_block), uint32_t(block_count - wave_first_block),
                                 uint32_t(padded_rows), uint32_t(tail_rows)};
        ++wave_count;
        wave_first_block = block_count;
    }
};

struct Piece {
    uint32_t slot;
    int64_t pair_start, rows;
};

}  // namespace

extern "C" {

int shrike_make_token_expert_pairs(const uint32_t *indices, const uint16_t *weights_f16, uint32_t query_count,
                                   uint32_t top_k, shrike_token_expert_pair *out_pairs) {
    SHRIKE_REQUIRE(out_pairs != nullptr && (uint64_t(query_count) * top_k == 0 || (indices && weights_f16)),
                   "makeTokenExpertPairs: NULL argument");
    for (uint32_t token = 0; token < query_count; ++token) {
        for (uint32_t rank = 0; rank < top_k; ++rank) {
            const size_t i = size_t(token) * top_k + rank;
            out_pairs[i] = {token, indices[i], rank, uint32_t(weights_f16[i])};
        }
    }
    return 0;
}

int shrike_group_pairs(const shrike_token_expert_pair *pairs, size_t pair_count, int64_t query_count,
                       int64_t top_k, int64_t num_experts, int64_t tile_expert_count,
                       const uint64_t *expert_sort_keys, size_t sort_key_count, shrike_grouped_routes *out) {
    if (!out || (pair_count != 0 && !pairs))
        return grouping_fail(out, EINVAL, 0, 0, "groupTokenExpertPairs: NULL argument");
    out->group_count = out->tile_count = 0;
    out->max_pairs_per_expert = out->max_pairs_per_tile = out->max_live_experts_per_tile = 0;
    out->error_value[0] = out->error_value[1] = 0;
    // the reference's checks, in its order (PrefillMoEGrouping.swift:277-320)
    if (query_count < 0)
        return grouping_fail(out, SHRIKE_GROUPING_INVALID_QUERY_COUNT, query_count, 0,
                             "queryCount must be non-negative, got %lld", (long long)query_count);
    if (top_k <= 0)
        return grouping_fail(out, SHRIKE_GROUPING_INVALID_TOP_K, top_k, 0, "topK must be positive, got %lld", (long long)top_k);
    if (num_experts <= 0)
        return grouping_fail(out, SHRIKE_GROUPING_INVALID_NUM_EXPERTS, num_experts, 0,
                             "numExperts must be positive, got %lld", (long long)num_experts);
    if (tile_expert_count < 1 || tile_expert_count > 16)
        return grouping_fail(out, SHRIKE_GROUPING_INVALID_TILE_EXPERT_COUNT, tile_expert_count, 0,
                             "tileExpertCount must be in 1...16, got %lld", (long long)tile_expert_count);
    if (expert_sort_keys && int64_t(sort_key_count) != num_experts)
        return grouping_fail(out, SHRIKE_GROUPING_EXPERT_SORT_KEY_COUNT_MISMATCH, num_experts, int64_t(sort_key_count),
                             "expected %lld expert sort keys, got %zu", (long long)num_experts, sort_key_count);
    // query_count * top_k cannot overflow for any pair_count that can match it
    const bool count_ok = query_count <= INT64_MAX / top_k && uint64_t(query_count * top_k) == pair_count;
    if (!count_ok)
        return grouping_fail(out, SHRIKE_GROUPING_PAIR_COUNT_MISMATCH,
                             query_count <= INT64_MAX / top_k ? query_count * top_k : INT64_MAX, int64_t(pair_count),
                             "expected %lld route pairs, got %zu",
                             (long long)(query_count <= INT64_MAX / top_k ? query_count * top_k : INT64_MAX), pair_count);
    if (!out->sorted_pairs || !out->per_expert_offsets || !out->per_expert_counts || !out->groups || !out->tiles)
        return grouping_fail(out, EINVAL, 0, 0, "groupTokenExpertPairs: an output array is NULL");

    std::vector<uint8_t> seen(pair_count, 0);  // (token, rank) is dense in [0, queryCount * topK)
    for (size_t i = 0; i < pair_count; ++i) {
        const shrike_token_expert_pair &p = pairs[i];
        if (!(int64_t(p.token) < query_count))
            return grouping_fail(out, SHRIKE_GROUPING_TOKEN_OUT_OF_RANGE, p.token, 0, "route token %u is out of range", p.token);
        if (!(int64_t(p.rank) < top_k))
            return grouping_fail(out, SHRIKE_GROUPING_RANK_OUT_OF_RANGE, p.rank, 0, "route rank %u is out of range", p.rank);
        if (!(int64_t(p.expert) < num_experts))
            return grouping_fail(out, SHRIKE_GROUPING_EXPERT_OUT_OF_RANGE, p.expert, 0, "route expert %u is out of range", p.expert);
        uint8_t &mark = seen[size_t(p.token) * size_t(top_k) + p.rank];
        if (mark)
            return grouping_fail(out, SHRIKE_GROUPING_DUPLICATE_TOKEN_RANK, p.token, p.rank,
                                 "duplicate route pair for token %u, rank %u", p.token, p.rank);
        mark = 1;
    }

    // The reference sorts by (sort key, expert, token, rank). (token, rank) is unique, so the
    // order is total and a counting sort over experts of the token-major pairs gives the same
    // permutation: place every pair at its (token, rank) position, count per expert, then lay
    // the experts out in (sort key, expert) order.
    const size_t E = size_t(num_experts);
    std::vector<uint32_t> by_position(pair_count);
    for (size_t i = 0; i < pair_count; ++i) by_position[size_t(pairs[i].token) * size_t(top_k) + pairs[i].rank] = uint32_t(i);
    std::fill(out->per_expert_counts, out->per_expert_counts + E, 0u);
    std::fill(out->per_expert_offsets, out->per_expert_offsets + E, UINT32_MAX);
    for (size_t i = 0; i < pair_count; ++i) ++out->per_expert_counts[pairs[i].expert];
    std::vector<uint32_t> expert_order;
    expert_order.reserve(std::min(E, pair_count));
    for (size_t e = 0; e < E; ++e)
        if (out->per_expert_counts[e]) expert_order.push_back(uint32_t(e));
    if (expert_sort_keys)
        std::stable_sort(expert_order.begin(), expert_order.end(),
                         [&](uint32_t l, uint32_t r) { return expert_sort_keys[l] < expert_sort_keys[r]; });
    std::vector<uint32_t> cursor(E, 0);
    uint32_t at = 0;
    for (uint32_t e : expert_order) {
        const uint32_t count = out->per_expert_counts[e];
        out->per_expert_offsets[e] = at;
        cursor[e] = at;
        out->groups[out->group_count++] = {e, at, count};
        out->max_pairs_per_expert = std::max(out->max_pairs_per_expert, count);
        at += count;
    }
    for (size_t pos = 0; pos < pair_count; ++pos) {
        const shrike_token_expert_pair &p = pairs[by_position[pos]];
        out->sorted_pairs[cursor[p.expert]++] = p;
    }
    for (uint32_t g = 0; g < out->group_count;) {
        const uint32_t end = uint32_t(std::min<int64_t>(out->group_count, int64_t(g) + tile_expert_count));
        const shrike_moe_group &first = out->groups[g], &last = out->groups[end - 1];
        const shrike_moe_tile tile = {g, end - g, first.pair_start, last.pair_start + last.pair_count - first.pair_start};
        out->tiles[out->tile_count++] = tile;
        out->max_pairs_per_tile = std::max(out->max_pairs_per_tile, tile.pair_count);
        out->max_live_experts_per_tile = std::max(out->max_live_experts_per_tile, tile.group_count);
        g = end;
    }
    return SHRIKE_GROUPING_OK;
}

int shrike_sweep_order_resident_first_balanced(const uint32_t *experts, const int64_t *rows, const int64_t *last_row,
                                               size_t count, const uint8_t *resident, size_t resident_count,
                                               int64_t slots, int64_t tile_width, uint32_t *out_order,
                                               size_t *out_count) {
    SHRIKE_REQUIRE(out_order && out_count && (count == 0 || (experts && rows && last_row)), "sweep order: NULL argument");
    SHRIKE_REQUIRE(tile_width > 0, "sweep order: tileWidth must be positive, got %lld", (long long)tile_width);
    std::unordered_map<uint32_t, int64_t> rows_of, last_of;
    for (size_t i = 0; i < count; ++i) {
        SHRIKE_REQUIRE(last_of.emplace(experts[i], last_row[i]).second, "sweep order: expert %u listed twice", experts[i]);
        rows_of.emplace(experts[i], rows[i]);
    }
    const RowsOf rows_fn{rows_of};
    // PrefillMoEGrouping.swift:107-119: last row, then rows, then id, all ascending
    std::vector<uint32_t> ranked(experts, experts + count);
    std::sort(ranked.begin(), ranked.end(), [&](uint32_t l, uint32_t r) {
        const int64_t ll = last_of[l], rl = last_of[r];
        if (ll != rl) return ll < rl;
        const int64_t lr = rows_fn(l), rr = rows_fn(r);
        if (lr != rr) return lr < rr;
        return l < r;
    });
    std::vector<uint32_t> res, absent;
    for (uint32_t e : ranked) ((size_t(e) < resident_count && resident && resident[e]) ? res : absent).push_back(e);
    const size_t width = size_t(tile_width);
    std::vector<uint32_t> order;
    if (res.empty() || absent.empty()) {
        order = fallback_order(res, absent, rows_fn, width);
    } else {
        const int64_t rc = int64_t(res.size()), ac = int64_t(absent.size());
        const int64_t tile_count = (rc + ac + tile_width - 1) / tile_width;
        int64_t head = 0;
        while (head < tile_count) {  // :153-160
            const int64_t remaining = tile_count - head;
            const int64_t mixed_misses = (ac + remaining - 1) / remaining;
            if (rc - tile_width * head <= slots - 6 * mixed_misses) break;  // residentFirstHeadFactor
            ++head;
        }
        const int64_t mixed = tile_count - head;
        if (mixed <= 0) {
            order = fallback_order(res, absent, rows_fn, width);
        } else {
            const size_t head_n = std::min(res.size(), size_t(tile_width * head));
            order.assign(res.begin(), res.begin() + ptrdiff_t(head_n));
            const std::vector<uint32_t> rest(res.begin() + ptrdiff_t(head_n), res.end());
            std::vector<std::vector<uint32_t>> bins{size_t(mixed)};
            for (int64_t t = 0; t < mixed; ++t) {
                const int64_t lo = t * ac / mixed, hi = (t + 1) * ac / mixed;
                if (lo < hi) bins[size_t(t)].assign(absent.begin() + lo, absent.begin() + hi);
            }
            pack_into(rest, bins, rows_fn, width);
            for (auto &b : bins) order.insert(order.end(), b.begin(), b.end());
        }
    }
    std::copy(order.begin(), order.end(), out_order);
    *out_count = order.size();
    return 0;
}

void shrike_expert_sort_keys(const uint32_t *order, size_t count, size_t num_experts, uint64_t *out_keys) {
    for (size_t e = 0; e < num_experts; ++e) out_keys[e] = uint64_t(count);
    for (size_t rank = 0; rank < count; ++rank)
        if (size_t(order[rank]) < num_experts) out_keys[order[rank]] = uint64_t(rank);
}

int shrike_plan_expert_waves(const shrike_expert_pair_range *ranges, size_t range_count, const uint32_t *bound_experts,
                             size_t bound_count, int64_t staging_rows, int64_t row_tile, int64_t tail_tile,
                             shrike_routed_expert_block *blocks, size_t block_capacity, size_t *block_count,
                             shrike_routed_expert_wave *waves, size_t wave_capacity, size_t *wave_count) {
    SHRIKE_REQUIRE(block_count && wave_count && (range_count == 0 || ranges) && (bound_count == 0 || bound_experts),
                   "planExpertWaves: NULL argument");
    SHRIKE_REQUIRE((block_capacity == 0 || blocks) && (wave_capacity == 0 || waves), "planExpertWaves: NULL output array");
    *block_count = *wave_count = 0;
    const bool tailed = tail_tile != 0;
    if (tailed) {  // PrefillGroupedRoutedMoE.swift:109-116, :165-168
        SHRIKE_REQUIRE(row_tile == kBodyTile, "a tail tile packs %lld-row bodies; rowTile %lld cannot combine with it",
                       (long long)kBodyTile, (long long)row_tile);
        SHRIKE_REQUIRE(tail_tile == kTailTile, "tail tile %lld is not %lld", (long long)tail_tile, (long long)kTailTile);
    }
    const int64_t tile = tailed ? kBodyTile : row_tile;
    SHRIKE_REQUIRE(tile > 0, "rowTile must be positive, got %lld", (long long)tile);
    SHRIKE_REQUIRE(staging_rows >= tile && staging_rows % tile == 0,
                   "%lld staging rows is not a positive multiple of %lld", (long long)staging_rows, (long long)tile);
    std::unordered_map<uint32_t, uint32_t> slot_of;
    for (size_t i = 0; i < bound_count; ++i) slot_of.emplace(bound_experts[i], uint32_t(i));

    Planner plan{blocks, block_capacity, waves, wave_capacity};
    if (!tailed) {
        int64_t cursor = 0;
        auto close = [&]() {
            if (plan.block_count == plan.wave_first_block) return;
            plan.add_wave(cursor, 0);
            cursor = 0;
        };
        for (size_t r = 0; r < range_count; ++r) {
            const shrike_expert_pair_range &range = ranges[r];
            if (range.pair_count <= 0) continue;
            auto slot = slot_of.find(range.expert);
            SHRIKE_REQUIRE(slot != slot_of.end(), "expert %u is not bound in the tile", range.expert);
            int64_t consumed = 0;
            while (consumed < range.pair_count) {
                if (cursor == staging_rows) close();
                const int64_t rows = std::min(range.pair_count - consumed, staging_rows - cursor);
                plan.add_block(slot->second, range.pair_start + consumed, rows, cursor, cursor / tile);
                cursor += (rows + tile - 1) / tile * tile;
                consumed += rows;
            }
        }
        close();
    } else {
        // :160-241: bodies first, then 32-row tail tiles for remainders of at most 32 rows
        std::vector<Piece> body_pieces, tail_pieces;
        int64_t used = 0;
        auto close = [&]() {
            if (body_pieces.empty() && tail_pieces.empty()) return;
            int64_t cursor = 0;
            for (const Piece &p : body_pieces) {
                plan.add_block(p.slot, p.pair_start, p.rows, cursor, cursor / kBodyTile);
                cursor += (p.rows + kBodyTile - 1) / kBodyTile * kBodyTile;
            }
            const int64_t body_padded = cursor;
            for (size_t i = 0; i < tail_pieces.size(); ++i) {
                plan.add_block(tail_pieces[i].slot, tail_pieces[i].pair_start, tail_pieces[i].rows, cursor, int64_t(i));
                cursor += kTailTile;
            }
            plan.add_wave(cursor, cursor - body_padded);
            body_pieces.clear();
            tail_pieces.clear();
            used = 0;
        };
        auto padded_cost = [](int64_t rows) {
            const int64_t rem = rows % kBodyTile;
            return rows - rem + (rem == 0 ? 0 : rem <= kTailTile ? kTailTile : kBodyTile);
        };
        auto place = [&](uint32_t slot, int64_t pair_start, int64_t rows) {
            const int64_t rem = rows % kBodyTile;
            const int64_t body_rows = rem > kTailTile ? rows : rows - rem;
            if (body_rows > 0) body_pieces.push_back({slot, pair_start, body_rows});
            if (rem > 0 && rem <= kTailTile) tail_pieces.push_back({slot, pair_start + body_rows, rem});
            used += padded_cost(rows);
        };
        for (size_t r = 0; r < range_count; ++r) {
            const shrike_expert_pair_range &range = ranges[r];
            if (range.pair_count <= 0) continue;
            auto slot = slot_of.find(range.expert);
            SHRIKE_REQUIRE(slot != slot_of.end(), "expert %u is not bound in the tile", range.expert);
            int64_t consumed = 0;
            while (consumed < range.pair_count) {
                const int64_t remaining = range.pair_count - consumed;
                const int64_t available = staging_rows - used;
                if (used + padded_cost(remaining) <= staging_rows) {
                    place(slot->second, range.pair_start + consumed, remaining);
                    consumed += remaining;
                    continue;
                }
                const int64_t cut = available / kBodyTile * kBodyTile + (available % kBodyTile >= kTailTile ? kTailTile : 0);
                if (cut > 0) {
                    place(slot->second, range.pair_start + consumed, cut);
                    consumed += cut;
                }
                close();
            }
        }
        close();
    }
    *block_count = plan.block_count;
    *wave_count = plan.wave_count;
    if (plan.block_count > block_capacity || plan.wave_count > wave_capacity) {
        set_error("planExpertWaves: needs %zu blocks and %zu waves", plan.block_count, plan.wave_count);
        return ENOSPC;
    }
    return 0;
}

int shrike_row_tile_table(const shrike_routed_expert_block *blocks, size_t block_count, uint32_t padded_rows,
                          uint32_t row_tile, uint32_t *table) {
    SHRIKE_REQUIRE(row_tile > 0 && (block_count == 0 || blocks) && (padded_rows < row_tile || table), "rowTileTable: bad argument");
    const uint32_t tiles = padded_rows / row_tile;
    std::fill(table, table + tiles, 0u);
    for (size_t i = 0; i < block_count; ++i) {
        const uint32_t first = blocks[i].row_tile_start, n = (blocks[i].rows + row_tile - 1) / row_tile;
        SHRIKE_REQUIRE(uint64_t(first) + n <= tiles, "rowTileTable: block %zu leaves the wave", i);
        for (uint32_t t = first; t < first + n; ++t) table[t] = uint32_t(i);
    }
    return 0;
}

int shrike_row_tile_tables(const shrike_routed_expert_block *blocks, size_t block_count, uint32_t padded_rows,
                           uint32_t tail_rows, uint32_t *gather, uint32_t *body, uint32_t *tail) {
    SHRIKE_REQUIRE(tail_rows <= padded_rows && (block_count == 0 || blocks), "rowTileTables: bad argument");
    const uint32_t body_rows = padded_rows - tail_rows;
    const uint32_t n_gather = padded_rows / kTailTile, n_body = body_rows / kBodyTile, n_tail = tail_rows / kTailTile;
    SHRIKE_REQUIRE((!n_gather || gather) && (!n_body || body) && (!n_tail || tail), "rowTileTables: NULL table");
    std::fill(gather, gather + n_gather, 0u);
    std::fill(body, body + n_body, 0u);
    std::fill(tail, tail + n_tail, 0u);
    for (size_t i = 0; i < block_count; ++i) {
        const uint32_t start = blocks[i].staging_row;
        const bool is_tail = start >= body_rows;
        const uint32_t padded = is_tail ? uint32_t(kTailTile) : (blocks[i].rows + uint32_t(kBodyTile) - 1) / uint32_t(kBodyTile) * uint32_t(kBodyTile);
        SHRIKE_REQUIRE(uint64_t(start) + padded <= padded_rows, "rowTileTables: block %zu leaves the wave", i);
        for (uint32_t row = start; row < start + padded; row += uint32_t(kTailTile)) gather[row / kTailTile] = uint32_t(i);
        if (is_tail) {
            SHRIKE_REQUIRE(blocks[i].row_tile_start < n_tail, "rowTileTables: tail block %zu leaves the tail region", i);
            tail[blocks[i].row_tile_start] = uint32_t(i);
        } else {
            for (uint32_t t = start / kBodyTile; t < (start + padded) / kBodyTile; ++t) body[t] = uint32_t(i);
        }
    }
    return 0;
}

}  // extern "C"
