"""CPU restatement of the reference's host-side integer logic around the routed-expert
path. TEST INFRASTRUCTURE ONLY: imported by tests/ (and nothing in the product);
the shipped implementation is the C++ in shrike_amd/csrc/host_logic.cpp and
slot_cache.cpp, which the tests compare against these functions.

Every function follows one reference function (cited in its docstring) and is pinned
in tests/test_host_logic_oracle.py, tests/test_packed_layout.py, tests/test_tile_scheduler.py,
tests/test_prefetch_ring.py and tests/test_slot_cache_landings.py by the vectors the
reference's own unit tests hold.
All arithmetic here is integer; results are compared for equality.
"""
from __future__ import annotations

from dataclasses import dataclass, field

U32_MAX = 0xFFFFFFFF

ALLOWED_SLOTS = [8, 16, 24, 32, 64, 96, 128, 160, 192, 224, 256]
DEFAULT_BUDGET = 8 << 30


# ----------------------------------------------------------------------- budget

def parse_budget_bytes(text: str):
    """RuntimeConfiguration.parseBudgetBytes,
    sources/Shrike/Runtime/Configuration/RuntimeConfiguration.swift:111-129."""
    raw = text.strip(" ").upper()
    if not raw:
        return None
    for suffix, scale in (("GIB", 1 << 30), ("MIB", 1 << 20), ("KIB", 1 << 10), ("GB", 1 << 30),
                          ("MB", 1 << 20), ("KB", 1 << 10), ("G", 1 << 30), ("M", 1 << 20), ("K", 1 << 10)):
        if raw.endswith(suffix):
            number = raw[: -len(suffix)].strip(" ")
            value = _swift_double(number)
            if value is None or not value > 0:
                return None
            b = value * scale
            if b != b or b in (float("inf"), float("-inf")) or b < 1 or not b < float(2**63 - 1):
                return None
            return int(b)
    if not _is_swift_int(raw):
        return None
    plain = int(raw)
    if plain <= 0 or plain > 2**63 - 1:
        return None
    return plain


def _is_swift_int(s: str) -> bool:
    body = s[1:] if s[:1] in "+-" else s
    return body.isascii() and body.isdigit()


def _swift_double(s: str):
    # Swift's Double(String) accepts what strtod accepts when the whole string is consumed
    # and it holds no whitespace; "abc", "" and "2X" give nil.
    if not s or any(c.isspace() for c in s):
        return None
    allowed = set("0123456789+-.EINFATYXP")
    if any(c not in allowed for c in s.upper()):
        return None
    try:
        return float.fromhex(s) if s.upper().lstrip("+-").startswith("0X") else float(s)
    except ValueError:
        return None


def expert_cache_slots(expert_stride_bytes: int, layers: int, budget_bytes: int = DEFAULT_BUDGET) -> int:
    """RuntimeConfiguration.expertCacheSlots, RuntimeConfiguration.swift:137-149: the allowed
    count nearest to budget / (stride * layers); `min` keeps the first of equals."""
    if expert_stride_bytes <= 0 or layers <= 0:
        return ALLOWED_SLOTS[0]
    wanted = float(budget_bytes) / (float(expert_stride_bytes) * float(layers))
    best = ALLOWED_SLOTS[0]
    for s in ALLOWED_SLOTS[1:]:
        if abs(float(s) - wanted) < abs(float(best) - wanted):
            best = s
    return best


# ------------------------------------------------------------- pairs and grouping

@dataclass(frozen=True, order=False)
class Pair:
    """PrefillTokenExpertPair, sources/Shrike/Kernels/Prefill/MoE/PrefillRouter.swift:5-28."""
    token: int
    expert: int
    rank: int
    weight_bits: int

    def as_tuple(self):
        return (self.token, self.expert, self.rank, self.weight_bits)


def make_token_expert_pairs(indices, weight_bits, query_count: int, top_k: int):
    """PrefillRouter.makeTokenExpertPairs, PrefillRouter.swift:160-180 (token-major)."""
    assert len(indices) == query_count * top_k and len(weight_bits) == query_count * top_k
    return [Pair(t, int(indices[t * top_k + r]), r, int(weight_bits[t * top_k + r]))
            for t in range(query_count) for r in range(top_k)]


class GroupingError(Exception):
    def __init__(self, case: str, *values):
        super().__init__(case, *values)
        self.case = case
        self.values = values


@dataclass
class GroupedRoutes:
    sorted_pairs: list
    per_expert_offsets: list
    per_expert_counts: list
    groups: list  # (expert, pair_start, pair_count)
    tiles: list   # (group_start, group_count, pair_start, pair_count)
    query_count: int

    @property
    def max_pairs_per_expert(self):
        return max((g[2] for g in self.groups), default=0)

    @property
    def max_pairs_per_tile(self):
        return max((t[3] for t in self.tiles), default=0)

    @property
    def max_live_experts_per_tile(self):
        return max((t[1] for t in self.tiles), default=0)


def group_token_expert_pairs(pairs, query_count, top_k, num_experts, tile_expert_count=16,
                             expert_sort_keys=None) -> GroupedRoutes:
    """PrefillMoEGrouping.groupTokenExpertPairs,
    sources/Shrike/Kernels/Prefill/MoE/PrefillMoEGrouping.swift:269-370: checks in the
    reference's order, sort by (sort key, expert, token, rank), offsets (U32_MAX when absent),
    counts, groups, tiles of at most tile_expert_count groups."""
    if query_count < 0:
        raise GroupingError("invalidQueryCount", query_count)
    if top_k <= 0:
        raise GroupingError("invalidTopK", top_k)
    if num_experts <= 0:
        raise GroupingError("invalidNumExperts", num_experts)
    if not 1 <= tile_expert_count <= 16:
        raise GroupingError("invalidTileExpertCount", tile_expert_count)
    if expert_sort_keys is not None and len(expert_sort_keys) != num_experts:
        raise GroupingError("expertSortKeyCountMismatch", num_experts, len(expert_sort_keys))
    if len(pairs) != query_count * top_k:
        raise GroupingError("pairCountMismatch", query_count * top_k, len(pairs))
    seen = set()
    for p in pairs:
        if not p.token < query_count:
            raise GroupingError("tokenOutOfRange", p.token)
        if not p.rank < top_k:
            raise GroupingError("rankOutOfRange", p.rank)
        if not p.expert < num_experts:
            raise GroupingError("expertOutOfRange", p.expert)
        if (p.token, p.rank) in seen:
            raise GroupingError("duplicateTokenRank", p.token, p.rank)
        seen.add((p.token, p.rank))

    def key(p):
        lead = (expert_sort_keys[p.expert],) if expert_sort_keys is not None else ()
        return lead + (p.expert, p.token, p.rank)

    s = sorted(pairs, key=key)  # (token, rank) is unique, so the order is total
    offsets = [U32_MAX] * num_experts
    counts = [0] * num_experts
    groups = []
    i = 0
    while i < len(s):
        e, start = s[i].expert, i
        while i < len(s) and s[i].expert == e:
            i += 1
        offsets[e], counts[e] = start, i - start
        groups.append((e, start, i - start))
    tiles = []
    g = 0
    while g < len(groups):
        end = min(len(groups), g + tile_expert_count)
        first, last = groups[g], groups[end - 1]
        tiles.append((g, end - g, first[1], last[1] + last[2] - first[1]))
        g = end
    return GroupedRoutes(s, offsets, counts, groups, tiles, query_count)


# ---------------------------------------------------------------------- sweep order

HEAD_FACTOR = 6      # PrefillMoEGrouping.swift:96
FALLBACK_TAIL = 96   # PrefillMoEGrouping.swift:101


def _ranked(rows, last_row):
    """PrefillSweepOrder.residentFirstRanked, PrefillMoEGrouping.swift:107-119."""
    return sorted(last_row.keys(), key=lambda e: (last_row.get(e, 0), rows.get(e, 0), e))


def _heaviest_first(experts, rows):
    return sorted(experts, key=lambda e: (-rows.get(e, 0), e))


def _pack_by_rows(experts, rows, tile_width):
    """packByRows, PrefillMoEGrouping.swift:203-226: heaviest first into the lightest bin
    that still has room, ties to the lower bin."""
    if not experts:
        return []
    n = (len(experts) + tile_width - 1) // tile_width
    totals, bins = [0] * n, [[] for _ in range(n)]
    for e in _heaviest_first(experts, rows):
        best, best_total = -1, None
        for i in range(n):
            if len(bins[i]) < tile_width and (best_total is None or totals[i] < best_total):
                best, best_total = i, totals[i]
        if best < 0:
            break
        bins[best].append(e)
        totals[best] += rows.get(e, 0)
    return [e for b in bins for e in b]


def _pack_by_rows_into(experts, preseeded, rows, tile_width):
    """packByRows(_:into:), PrefillMoEGrouping.swift:234-261."""
    bins = [list(b) for b in preseeded]
    weights = [sum(rows.get(e, 0) for e in b) for b in bins]
    for e in _heaviest_first(experts, rows):
        best, best_w = -1, None
        for i in range(len(bins)):
            if len(bins[i]) < tile_width and (best_w is None or weights[i] < best_w):
                best, best_w = i, weights[i]
        if best < 0:
            break
        bins[best].append(e)
        weights[best] += rows.get(e, 0)
    return bins


def _fallback_order(resident_group, absent_group, rows, tile_width):
    """residentFirstFallbackOrder, PrefillMoEGrouping.swift:179-190."""
    tail = min(FALLBACK_TAIL, len(absent_group))
    head = len(absent_group) - tail
    return (_pack_by_rows(resident_group, rows, tile_width)
            + _pack_by_rows(absent_group[:head], rows, tile_width)
            + _pack_by_rows(absent_group[head:], rows, tile_width))


def resident_first_balanced(rows: dict, last_row: dict, resident, slots: int, tile_width: int):
    """PrefillSweepOrder.residentFirstBalanced, PrefillMoEGrouping.swift:131-177."""
    ranked = _ranked(rows, last_row)
    res = [e for e in ranked if e < len(resident) and resident[e]]
    absent = [e for e in ranked if not (e < len(resident) and resident[e])]
    if not res or not absent:
        return _fallback_order(res, absent, rows, tile_width)
    tile_count = (len(res) + len(absent) + tile_width - 1) // tile_width
    head = 0
    while head < tile_count:
        remaining = tile_count - head
        mixed_misses = (len(absent) + remaining - 1) // remaining
        if len(res) - tile_width * head <= slots - HEAD_FACTOR * mixed_misses:
            break
        head += 1
    head_res, rest_res = res[: tile_width * head], res[tile_width * head:]
    mixed = tile_count - head
    if mixed <= 0:
        return _fallback_order(res, absent, rows, tile_width)
    bins = []
    for t in range(mixed):
        lo, hi = (t * len(absent)) // mixed, ((t + 1) * len(absent)) // mixed
        bins.append(absent[lo:hi] if lo < hi else [])
    filled = _pack_by_rows_into(rest_res, bins, rows, tile_width)
    return head_res + [e for b in filled for e in b]


def expert_sort_keys(order, num_experts: int):
    """PrefillSweepOrder.expertSortKeys, PrefillMoEGrouping.swift:196-202."""
    keys = [len(order)] * num_experts
    for rank, e in enumerate(order):
        if e < num_experts:
            keys[e] = rank
    return keys


# --------------------------------------------------------------------- wave planner

ROW_TILE = 64   # MPPPrefillInt4QMM.tileM
TAIL_TILE = 32


class PlanError(Exception):
    pass


@dataclass
class Wave:
    blocks: list  # (slot, pair_start, rows, staging_row, row_tile_start)
    padded_rows: int
    tail_rows: int = 0

    @property
    def body_padded_rows(self):
        return self.padded_rows - self.tail_rows


def plan_expert_waves(ranges, bound_experts, staging_rows, row_tile=ROW_TILE, tail_tile=0):
    """PrefillGroupedRoutedMoE.planExpertWaves,
    sources/Shrike/Kernels/Prefill/MoE/PrefillGroupedRoutedMoE.swift:104-150 (and the tail
    variant :160-241). `ranges` are (expert, pair_start, pair_count); an expert's local slot
    is its position in `bound_experts`."""
    slot_of = {}
    for i, e in enumerate(bound_experts):
        slot_of.setdefault(e, i)
    if tail_tile != 0:
        if row_tile != ROW_TILE:
            raise PlanError("a tail tile packs 64-row bodies")
        return _plan_with_tail(ranges, slot_of, staging_rows, tail_tile)
    tile = row_tile
    if not (staging_rows >= tile and staging_rows % tile == 0):
        raise PlanError("stagingTooSmall")
    waves, blocks, cursor = [], [], 0

    def close():
        nonlocal blocks, cursor
        if blocks:
            waves.append(Wave(blocks, cursor))
            blocks, cursor = [], 0

    for expert, pair_start, pair_count in ranges:
        if pair_count <= 0:
            continue
        if expert not in slot_of:
            raise PlanError("expert %d is not bound in the tile" % expert)
        consumed = 0
        while consumed < pair_count:
            if cursor == staging_rows:
                close()
            rows = min(pair_count - consumed, staging_rows - cursor)
            blocks.append((slot_of[expert], pair_start + consumed, rows, cursor, cursor // tile))
            cursor += (rows + tile - 1) // tile * tile
            consumed += rows
    close()
    return waves


def _plan_with_tail(ranges, slot_of, staging_rows, tail_tile):
    body = ROW_TILE
    if tail_tile != TAIL_TILE:
        raise PlanError("tail tile is not 32")
    if not (staging_rows >= body and staging_rows % body == 0):
        raise PlanError("stagingTooSmall")
    waves, body_pieces, tail_pieces = [], [], []
    used = 0

    def close():
        nonlocal body_pieces, tail_pieces, used
        if not body_pieces and not tail_pieces:
            return
        blocks, cursor = [], 0
        for slot, ps, rows in body_pieces:
            blocks.append((slot, ps, rows, cursor, cursor // body))
            cursor += (rows + body - 1) // body * body
        body_padded = cursor
        for i, (slot, ps, rows) in enumerate(tail_pieces):
            blocks.append((slot, ps, rows, cursor, i))
            cursor += tail_tile
        waves.append(Wave(blocks, cursor, cursor - body_padded))
        body_pieces, tail_pieces, used = [], [], 0

    def padded_cost(rows):
        rem = rows % body
        return rows - rem + (0 if rem == 0 else tail_tile if rem <= tail_tile else body)

    def place(slot, ps, rows):
        nonlocal used
        rem = rows % body
        body_rows = rows if rem > tail_tile else rows - rem
        if body_rows > 0:
            body_pieces.append((slot, ps, body_rows))
        if 0 < rem <= tail_tile:
            tail_pieces.append((slot, ps + body_rows, rem))
        used += padded_cost(rows)

    for expert, pair_start, pair_count in ranges:
        if pair_count <= 0:
            continue
        if expert not in slot_of:
            raise PlanError("expert %d is not bound in the tile" % expert)
        consumed = 0
        while consumed < pair_count:
            remaining = pair_count - consumed
            available = staging_rows - used
            if used + padded_cost(remaining) <= staging_rows:
                place(slot_of[expert], pair_start + consumed, remaining)
                consumed += remaining
                continue
            cut = available // body * body + (tail_tile if available % body >= tail_tile else 0)
            if cut > 0:
                place(slot_of[expert], pair_start + consumed, cut)
                consumed += cut
            close()
    close()
    return waves


def row_tile_table(wave: Wave, row_tile=ROW_TILE):
    """rowTileTable, PrefillGroupedRoutedMoE.swift:272-283."""
    table = [0] * (wave.padded_rows // row_tile)
    for i, b in enumerate(wave.blocks):
        first, count = b[4], (b[2] + row_tile - 1) // row_tile
        for t in range(first, first + count):
            table[t] = i
    return table


def row_tile_tables(wave: Wave):
    """rowTileTables, PrefillGroupedRoutedMoE.swift:247-269: (gather, body, tail)."""
    body, tail = ROW_TILE, TAIL_TILE
    gather = [0] * (wave.padded_rows // tail)
    body_t = [0] * (wave.body_padded_rows // body)
    tail_t = [0] * (wave.tail_rows // tail)
    for i, b in enumerate(wave.blocks):
        start = b[3]
        is_tail = start >= wave.body_padded_rows
        padded = tail if is_tail else (b[2] + body - 1) // body * body
        for row in range(start, start + padded, tail):
            gather[row // tail] = i
        if is_tail:
            tail_t[b[4]] = i
        else:
            for t in range(start // body, (start + padded) // body):
                body_t[t] = i
    return gather, body_t, tail_t


# ----------------------------------------------------------------------- slot pool

EMPTY, LOADING, RESIDENT = 0, 1, 2


def residency_word(state: int, cell: int) -> int:
    """ExpertResidencyEntry as the 64-bit word the kernels read,
    sources/Shrike/Infrastructure/Streaming/ExpertResidencyTable.swift:4-18 and the publish
    rule of PreadExpertStreamer.swift:1143-1148 (an empty entry names the sentinel cell)."""
    slot = U32_MAX if state == EMPTY else cell & U32_MAX
    return (state << 32) | slot


@dataclass
class CachePlan:
    experts: list
    assigned_slots: list
    assigned_generations: list
    misses: list  # indices into experts
    hits: int
    layer: int = 0
    adopted: list = field(default_factory=list)  # indices into experts
    freed_cells: dict = field(default_factory=dict)  # expert -> the pool cell its swap gave back
    assigned_cells: list = field(default_factory=list)


class CellArena:
    """ExpertCellArena's generations (ExpertCellArena.swift:95-104): one clock for all cells."""

    def __init__(self, cell_count: int):
        assert cell_count > 0
        self.cell_count = cell_count
        self.generations = [0] * cell_count
        self.clock = 0

    def cell_generation(self, cell):
        return self.generations[cell]

    def bump(self, cell):
        self.clock += 1
        self.generations[cell] = self.clock
        return self.clock


class ClaimRefusedByPool(Exception):
    """PrefetchClaimRefused as beginPrefetch throws it (PreadExpertStreamer.swift:1050-1053)."""

    def __init__(self, expert, cell):
        super().__init__(f"prefetch claim refused: expert {expert}, cell {cell}")
        self.expert, self.cell = expert, cell


@dataclass
class SlotCache:
    """The slot bookkeeping of PreadExpertStreamer (PreadExpertStreamer.swift:405-543,
    :676-767, :1085-1148) without the file reads: hits, victim choice (aging LFU then LRU, or
    SLRU), loading/resident states, arena-wide cell generations, pins, statistics and the
    residency words; the landings a prefetch ring claims (:815-852, :1010-1018), their
    adoption by a plan (:499-515) and the overflow slots of a decode route (:860-1002)."""
    slot_count: int
    experts_per_layer: int
    first_cell: int = 0
    slru_share: float | None = None  # None = aging LFU
    arena: CellArena | None = None  # None = an arena of its own

    def __post_init__(self):
        n, e = self.slot_count, max(1, self.experts_per_layer)
        if self.arena is None:
            self.arena = CellArena(self.first_cell + n)
        assert self.first_cell + n <= self.arena.cell_count
        self.slot_cell = [self.first_cell + s for s in range(n)]
        self.landings = {}  # expert -> [cell, resident, generation]
        self.overflow_probation = set()
        self.slot_expert = [-1] * n
        self.slot_last_use = [0] * n
        self.slot_state = [EMPTY] * n
        self.slot_pins = [0] * n
        self.slot_protected = [False] * n
        self.protected_count = 0
        # ExpertEvictionPolicy.protectedCapacity, Model.swift:26-33 (rounds half away from zero)
        self.protected_capacity = 0 if self.slru_share is None else max(1, int(self.slru_share * n + 0.5))
        self.use_count = [0] * e
        self.load_count = [0] * e
        self.use_clock = 0
        self.words = [residency_word(EMPTY, 0)] * self.experts_per_layer
        self.stats = dict(plans=0, requested=0, hits=0, misses=0, evictions=0, reloads=0,
                          read_operations=0, load_batches=0, peak_loading=0)

    def cell(self, slot):
        """cellIndexUnlocked, PreadExpertStreamer.swift:1135-1137."""
        return self.slot_cell[slot]

    def _generation(self, slot):
        return self.arena.cell_generation(self.slot_cell[slot])

    def _slot_of_cell(self, cell):
        return self.slot_cell.index(cell) if cell in self.slot_cell else None

    def owns_cell(self, cell):
        return cell in self.slot_cell

    def _demote(self, slot):
        if self.slot_protected[slot]:
            self.slot_protected[slot] = False
            self.protected_count -= 1

    def _record_expert_load(self, e):
        """recordExpertLoadsUnlocked, PreadExpertStreamer.swift:1171-1179."""
        if 0 <= e < len(self.load_count):
            if self.load_count[e] > 0:
                self.stats["reloads"] += 1
            self.load_count[e] += 1

    def _publish(self, expert, cell, state):
        if 0 <= expert < self.experts_per_layer:
            self.words[expert] = residency_word(state, cell)

    def _should_evict(self, lhs, rhs):
        """shouldEvictSlot, PreadExpertStreamer.swift:728-742."""
        le, re = self.slot_expert[lhs], self.slot_expert[rhs]
        if le < 0 or re < 0:
            return le < re
        if self.slru_share is not None:
            if self.slot_protected[lhs] != self.slot_protected[rhs]:
                return not self.slot_protected[lhs]
            return self.slot_last_use[lhs] < self.slot_last_use[rhs]
        lc = self.use_count[le] if le < len(self.use_count) else 0
        rc = self.use_count[re] if re < len(self.use_count) else 0
        if lc != rc:
            return lc < rc
        return self.slot_last_use[lhs] < self.slot_last_use[rhs]

    def _select_victims(self, miss_count, reserved, protected=None):
        """selectVictimSlots, PreadExpertStreamer.swift:676-705."""
        victims, eligible = [], 0
        for slot in range(self.slot_count):
            if reserved[slot] or self.slot_state[slot] == LOADING or self.slot_pins[slot] != 0:
                continue
            e = self.slot_expert[slot]
            if protected is not None and 0 <= e < len(protected) and protected[e]:
                continue
            eligible += 1
            if len(victims) < miss_count:
                at = len(victims)
                victims.append(slot)
                while at > 0 and self._should_evict(slot, victims[at - 1]):
                    victims[at] = victims[at - 1]
                    at -= 1
                victims[at] = slot
            elif victims and self._should_evict(slot, victims[-1]):
                at = len(victims) - 1
                while at > 0 and self._should_evict(slot, victims[at - 1]):
                    victims[at] = victims[at - 1]
                    at -= 1
                victims[at] = slot
        return victims if miss_count <= eligible else None

    def _promote(self, slot, clock):
        """promoteToProtected, PreadExpertStreamer.swift:708-720."""
        self.slot_protected[slot] = True
        self.protected_count += 1
        if self.protected_count <= self.protected_capacity:
            return
        oldest = -1
        for c in range(self.slot_count):
            if self.slot_protected[c] and c != slot:
                if oldest < 0 or self.slot_last_use[c] < self.slot_last_use[oldest]:
                    oldest = c
        if oldest < 0:
            return
        self.slot_protected[oldest] = False
        self.protected_count -= 1
        self.slot_last_use[oldest] = clock

    def plan(self, experts, layer=0, avoiding_slots=(), protected_experts=None, misses_counted=None,
             gpu_missed_experts=None, leased_landings=()):
        """makeExpertCachePlan, PreadExpertStreamer.swift:405-543; None when unplaceable."""
        assert len(experts) <= self.slot_count
        avoiding = {s for s in avoiding_slots if 0 <= s < self.slot_count}
        reserved = [False] * self.slot_count
        clock = self.use_clock + 1
        if self.stats["plans"] > 0 and self.stats["plans"] % 1024 == 0:
            self.use_count = [c >> 1 for c in self.use_count]
        for s in range(self.slot_count):
            if self.slot_state[s] == LOADING:
                reserved[s] = True
        assigned = [-1] * len(experts)
        miss_count = 0
        for i, e in enumerate(experts):
            for s in range(self.slot_count):
                if not reserved[s] and self.slot_state[s] == RESIDENT and self.slot_expert[s] == e:
                    assigned[i] = s
                    reserved[s] = True
                    break
            if assigned[i] == -1:
                miss_count += 1
        for s in avoiding:
            reserved[s] = True
        victims = []
        if miss_count > 0:
            victims = self._select_victims(miss_count, reserved, protected_experts) if protected_experts is not None else None
            if victims is None:
                victims = self._select_victims(miss_count, reserved)
                if victims is None:
                    return None
        self.use_clock = clock
        for e in experts:
            if 0 <= e < len(self.use_count):
                self.use_count[e] += 1
        for s in assigned:
            if s >= 0:
                self.slot_last_use[s] = clock
        if self.slru_share is not None:
            for s in assigned:
                if s >= 0 and not self.slot_protected[s]:
                    if s in self.overflow_probation:
                        self.overflow_probation.discard(s)
                        continue
                    self._promote(s, clock)
        misses, v = [], 0
        adopted, freed = [], {}
        for i, e in enumerate(experts):
            if assigned[i] != -1:
                continue
            slot = victims[v]
            v += 1
            if self.slot_state[slot] == RESIDENT:
                self.stats["evictions"] += 1
            previous = self.slot_expert[slot]
            assigned[i] = slot
            reserved[slot] = True
            self._demote(slot)
            self.overflow_probation.discard(slot)
            cell = self.cell(slot)
            self.arena.bump(cell)
            if previous >= 0:
                self._publish(previous, cell, EMPTY)
            landing = self.landings.get(e) if e in leased_landings else None
            if landing is not None and landing[1]:
                del self.landings[e]
                freed[e] = cell
                self.slot_cell[slot] = landing[0]
                self.slot_expert[slot] = e
                self.slot_last_use[slot] = clock
                self.slot_state[slot] = RESIDENT
                self._record_expert_load(e)
                if gpu_missed_experts is not None and e in gpu_missed_experts:
                    adopted.append(i)
                continue
            self.slot_expert[slot] = e
            self.slot_last_use[slot] = clock
            self.slot_state[slot] = LOADING
            self._publish(e, cell, LOADING)
            misses.append(i)
        counted = len(misses) if misses_counted is None else misses_counted
        self.stats["plans"] += 1
        self.stats["requested"] += len(experts)
        self.stats["hits"] += len(experts) - counted
        self.stats["misses"] += counted
        self.stats["peak_loading"] = max(self.stats["peak_loading"], self.slot_state.count(LOADING))
        return CachePlan(list(experts), assigned, [self._generation(s) for s in assigned], misses,
                         len(experts) - len(misses), layer, adopted, freed, [self.cell(s) for s in assigned])

    def complete(self, plan: CachePlan):
        """markPlanMissesResident + the success leg of finishPlanExecution,
        PreadExpertStreamer.swift:1085-1105, :1070-1083, :1150-1179."""
        for i in plan.misses:
            if self._generation(plan.assigned_slots[i]) != plan.assigned_generations[i]:
                raise RuntimeError("expert-cache cell generation changed during expert load")
        for i in plan.misses:
            s = plan.assigned_slots[i]
            self.slot_state[s] = RESIDENT
            self.slot_expert[s] = plan.experts[i]
            self.slot_last_use[s] = self.use_clock
            self._publish(plan.experts[i], self.cell(s), RESIDENT)
        if plan.misses:
            self.stats["read_operations"] += len(plan.misses)
            self.stats["load_batches"] += 1
            for i in plan.misses:
                self._record_expert_load(plan.experts[i])

    def abandon(self, plan: CachePlan):
        """abandonExpertCachePlan / resetLoadingMissesUnlocked, PreadExpertStreamer.swift:1110-1128."""
        for i in plan.misses:
            s = plan.assigned_slots[i]
            if not (0 <= s < self.slot_count and self._generation(s) == plan.assigned_generations[i]
                    and self.slot_state[s] == LOADING):
                continue
            self.slot_state[s] = EMPTY
            self.slot_expert[s] = -1
            self._publish(plan.experts[i], self.cell(s), EMPTY)

    def load(self, experts, **kw):
        """loadExpertsCached, PreadExpertStreamer.swift:355-358."""
        p = self.plan(experts, **kw)
        if p is None:
            raise RuntimeError("unplaceable")
        self.complete(p)
        return p

    def pin(self, plan: CachePlan):
        """pin, PreadExpertStreamer.swift:744-767; raises on a stale plan."""
        for i, e in enumerate(plan.experts):
            s = plan.assigned_slots[i]
            if not (0 <= s < self.slot_count and self._generation(s) == plan.assigned_generations[i]
                    and self.slot_expert[s] == e and self.slot_state[s] != EMPTY):
                raise RuntimeError("expert-cache plan became stale before GPU pin")
        for s in plan.assigned_slots:
            self.slot_pins[s] += 1

    def unpin(self, slots, generations):
        """unpin, PreadExpertStreamer.swift:769-778."""
        for s, g in zip(slots, generations):
            if 0 <= s < self.slot_count and self._generation(s) == g:
                assert self.slot_pins[s] > 0
                self.slot_pins[s] -= 1

    def resident_experts(self):
        """residentExperts, PreadExpertStreamer.swift:807-813."""
        return sorted(e for e, st in zip(self.slot_expert, self.slot_state) if st == RESIDENT and e >= 0)

    def counts(self):
        return dict(resident=self.slot_state.count(RESIDENT), loading=self.slot_state.count(LOADING),
                    pinned=sum(1 for p in self.slot_pins if p > 0))

    # ---- landings (a prefetch ring's cells outside the pool)

    def claim_landing(self, expert, cell):
        """claimLanding, PreadExpertStreamer.swift:815-829."""
        if not (0 <= expert < self.experts_per_layer and 0 <= cell < self.arena.cell_count):
            return False
        if expert in self.landings or expert in self.slot_expert or any(l[0] == cell for l in self.landings.values()):
            return False
        self.landings[expert] = [cell, False, self.arena.bump(cell)]
        self._publish(expert, cell, LOADING)
        return True

    def complete_landing(self, expert, cell):
        """completeLanding, PreadExpertStreamer.swift:834-848."""
        landing = self.landings.get(expert)
        if landing is None or landing[0] != cell or landing[1] or self.arena.cell_generation(cell) != landing[2]:
            return False
        if expert in self.slot_expert:
            del self.landings[expert]
            return False
        landing[1] = True
        self._publish(expert, cell, RESIDENT)
        return True

    def drop_landing(self, expert, cell):
        """dropLanding, PreadExpertStreamer.swift:1010-1018 (failLanding, :850-852, is the same)."""
        landing = self.landings.get(expert)
        if landing is None or landing[0] != cell:
            return
        del self.landings[expert]
        if expert not in self.slot_expert:
            self._publish(expert, cell, EMPTY)

    fail_landing = drop_landing

    def claim_prefetch(self, experts, cells):
        """The claims of beginPrefetch, PreadExpertStreamer.swift:1034-1057."""
        if len(experts) != len(cells):
            raise ValueError("prefetch experts and cells differ in count")
        if any(not 0 <= e < self.experts_per_layer for e in experts):
            raise ValueError("invalid prefetched expert")
        if any(self.owns_cell(c) for c in cells):
            raise ValueError("a prefetch landing was offered a cell the pool owns")
        landed = []
        for e, c in zip(experts, cells):
            if not self.claim_landing(e, c):
                for pe, pc in landed:
                    self.drop_landing(pe, pc)
                raise ClaimRefusedByPool(e, c)
            landed.append((e, c))

    # ---- overflow slots (a decode route's misses the ring could not house)

    def reserve_overflow_slot(self, expert, protecting=()):
        """reserveOverflowSlot, PreadExpertStreamer.swift:860-893: the cell, or None."""
        if not 0 <= expert < self.experts_per_layer or expert in self.slot_expert:
            return None
        reserved = [st == LOADING for st in self.slot_state]
        for s in range(self.slot_count):
            if self.slot_state[s] == RESIDENT and self.slot_expert[s] in protecting:
                reserved[s] = True
        victims = self._select_victims(1, reserved)
        if victims is None:
            return None
        slot = victims[0]
        self.overflow_probation.add(slot)
        if self.slot_state[slot] == RESIDENT:
            self.stats["evictions"] += 1
        previous = self.slot_expert[slot]
        self._demote(slot)
        cell = self.cell(slot)
        self.arena.bump(cell)
        if previous >= 0:
            self._publish(previous, cell, EMPTY)
        self.slot_expert[slot] = expert
        self.slot_last_use[slot] = self.use_clock
        self.slot_state[slot] = LOADING
        self._publish(expert, cell, LOADING)
        return cell

    def mark_overflow_resident(self, expert, cell):
        """markOverflowResident, PreadExpertStreamer.swift:968-976."""
        slot = self._slot_of_cell(cell)
        if slot is None or self.slot_state[slot] != LOADING or self.slot_expert[slot] != expert:
            return
        self.slot_state[slot] = RESIDENT
        self.slot_last_use[slot] = self.use_clock
        self._publish(expert, cell, RESIDENT)

    def abandon_overflow_slot(self, expert, cell):
        """abandonOverflowSlot / emptyOverflowSlot, PreadExpertStreamer.swift:980-993."""
        slot = self._slot_of_cell(cell)
        if slot is None or self.slot_state[slot] != LOADING or self.slot_expert[slot] != expert:
            return
        self.slot_state[slot] = EMPTY
        self.slot_expert[slot] = -1
        self.overflow_probation.discard(slot)
        self._publish(expert, cell, EMPTY)

    def finish_agreed_reads(self, experts, cells, succeeded):
        """The completion of beginAgreedReads, PreadExpertStreamer.swift:936-964, :995-1002."""
        pool = [self.owns_cell(c) for c in cells]
        for e, c, in_pool in zip(experts, cells, pool):
            if succeeded:
                self.mark_overflow_resident(e, c) if in_pool else self.complete_landing(e, c)
            else:
                self.abandon_overflow_slot(e, c) if in_pool else self.drop_landing(e, c)
        if succeeded and experts:
            self.stats["read_operations"] += len(experts)
            self.stats["load_batches"] += 1
            for e, in_pool in zip(experts, pool):
                if in_pool:
                    self._record_expert_load(e)


# ------------------------------------------------------------- packed experts layout

LAYOUT_ALIGNMENT = 16384  # GTurboFormatV1.alignmentBytes, sources/ShrikeFormat/GTurboFormatV1.swift:7


class LayoutInvalid(Exception):
    """ShrikeFormatError.invalid(field:reason:)."""

    def __init__(self, field_: str, reason: str):
        super().__init__(f"{field_}: {reason}")
        self.field, self.reason = field_, reason


def _basename_fault(name: str):
    """GTurboPathValidator.validateBasename, sources/ShrikeFormat/GTurboFormatV1.swift:58-77."""
    if name == "" or name.startswith("/") or "\0" in name:
        return "unsafe relative path"
    if any(c in ("", ".", "..") for c in name.split("/")):
        return "non-canonical path"
    if "/" in name:
        return "expected basename"
    return None


def _is_int(v) -> bool:
    return isinstance(v, int) and not isinstance(v, bool)


def decode_packed_layout(data: bytes) -> dict:
    """GTurboPackedExpertsLayoutCodec.decode + GTurboV1StructuralValidator.validate
    (sources/ShrikeFormat/GTurboPackedExpertsLayoutV1.swift:65-164) and the runtime view of
    PackedExpertsLayoutReader.decode (sources/Shrike/Infrastructure/ModelIO/PackedExpertsLayout.swift:104-128):
    layers by id, experts by logical id. Raises LayoutInvalid with the reference's reason."""
    import json
    try:
        root = json.loads(data)
        stride, num_layers, per_layer = root["expertStride"], root["numLayers"], root["expertsPerLayer"]
        layers_in = root["layers"]
        if not (_is_int(stride) and stride >= 0 and _is_int(num_layers) and _is_int(per_layer)
                and isinstance(layers_in, list)):
            raise TypeError("mistyped top-level key")
        layers = []
        for lj in layers_in:
            experts = []
            for ej in lj["experts"]:
                tensors = {}
                for name, tj in ej["tensors"].items():
                    t = {"offset": tj["offset"], "size": tj["size"], "dtype": tj["dtype"], "shape": list(tj["shape"]),
                         "bits": tj.get("bits")}
                    if not (_is_int(t["offset"]) and t["offset"] >= 0 and _is_int(t["size"]) and t["size"] >= 0
                            and isinstance(t["dtype"], str) and all(_is_int(d) and 0 <= d <= U32_MAX for d in t["shape"])
                            and (t["bits"] is None or _is_int(t["bits"]))):
                        raise TypeError("mistyped tensor")
                    tensors[name] = t
                e = {"expert": ej.get("expert"), "physicalRank": ej.get("physicalRank"), "offset": ej["offset"],
                     "size": ej["size"], "tensors": tensors}
                if not (_is_int(e["offset"]) and e["offset"] >= 0 and _is_int(e["size"]) and e["size"] >= 0
                        and all(v is None or _is_int(v) for v in (e["expert"], e["physicalRank"]))):
                    raise TypeError("mistyped expert")
                experts.append(e)
            if not (_is_int(lj["layer"]) and isinstance(lj["file"], str)):
                raise TypeError("mistyped layer")
            layers.append({"layer": lj["layer"], "file": lj["file"], "experts": experts})
    except (ValueError, KeyError, TypeError, AttributeError) as exc:
        raise LayoutInvalid("packed_experts/layout.json", str(exc))

    if not (num_layers > 0 and per_layer > 0 and stride > 0 and stride % LAYOUT_ALIGNMENT == 0
            and len(layers) == num_layers):
        raise LayoutInvalid("layout", "invalid dimensions or stride")
    layer_ids, layer_files = set(), set()
    for layer in layers:
        lid = layer["layer"]
        if not (0 <= lid < num_layers) or lid in layer_ids:
            raise LayoutInvalid("layout.layers", "duplicate or invalid layer")
        layer_ids.add(lid)
        fault = _basename_fault(layer["file"])
        if fault:
            raise LayoutInvalid(f"layout.layers[{lid}].file", fault)
        key = "".join(chr(ord(c) + 32) if "A" <= c <= "Z" else c for c in layer["file"])
        if key == "layout.json":
            raise LayoutInvalid(f"layout.layers[{lid}].file", "reserved packed-expert filename")
        if key in layer_files:
            raise LayoutInvalid(f"layout.layers[{lid}].file", "duplicate layer filename")
        layer_files.add(key)
        experts = layer["experts"]
        if len(experts) not in (per_layer, 0):
            raise LayoutInvalid(f"layout.layers[{lid}].experts", "wrong expert count")
        explicit = [e["expert"] is not None for e in experts]
        if any(explicit) and not all(explicit):
            raise LayoutInvalid(f"layout.layers[{lid}].experts",
                                "expert ids must be either all explicit or all positional")
        logical_ids, ranks, offsets = set(), set(), set()
        for position, e in enumerate(experts):
            logical = e["expert"] if e["expert"] is not None else position
            physical = e["physicalRank"] if e["physicalRank"] is not None else logical
            if (not (0 <= logical < per_layer and 0 <= physical < per_layer) or logical in logical_ids
                    or physical in ranks or e["offset"] in offsets):
                raise LayoutInvalid(f"layout.layers[{lid}].experts", "duplicate or invalid expert mapping")
            logical_ids.add(logical), ranks.add(physical), offsets.add(e["offset"])
            if physical * stride >= 1 << 64:
                raise LayoutInvalid("expert.offset", "overflow")
            if not (e["offset"] == physical * stride and e["size"] == stride):
                raise LayoutInvalid(f"expert[{logical}]", "offset or size does not match physical rank")
            ranges = []
            for name, t in e["tensors"].items():
                if not (t["dtype"] in ("U32", "BF16") and name != "" and t["size"] > 0 and len(t["shape"]) > 0
                        and all(d > 0 for d in t["shape"]) and (t["bits"] is None or 0 < t["bits"] <= 32)):
                    raise LayoutInvalid(f"expert[{logical}].tensors.{name}", "invalid dtype or shape")
                end = t["offset"] + t["size"]
                if end >= 1 << 64:
                    raise LayoutInvalid(f"tensor.{name}.range", "overflow")
                if end > e["size"]:
                    raise LayoutInvalid(f"expert[{logical}].tensors.{name}", "range exceeds expert blob")
                ranges.append((t["offset"], end, name))
            ranges.sort(key=lambda r: (r[0], r[1]))
            for a, b in zip(ranges, ranges[1:]):
                if a[1] > b[0]:
                    raise LayoutInvalid(f"expert[{logical}].tensors", f"overlapping ranges {a[2]} and {b[2]}")
            e["logical"], e["physical"] = logical, physical
    view = []
    for layer in sorted(layers, key=lambda l: l["layer"]):
        view.append({"layer": layer["layer"], "file": layer["file"],
                     "experts": sorted(layer["experts"], key=lambda e: e["logical"])})
    return {"expertStride": stride, "numLayers": num_layers, "expertsPerLayer": per_layer, "layers": view}


def cross_validate_layout(layout: dict, num_layers: int, per_layer: int, stride: int, file_sizes: dict) -> None:
    """GTurboV1StructuralValidator.crossValidate, GTurboPackedExpertsLayoutV1.swift:177-199."""
    if (num_layers, per_layer, stride) != (layout["numLayers"], layout["expertsPerLayer"], layout["expertStride"]):
        raise LayoutInvalid("manifest/layout", "dimension mismatch")
    layer_size = layout["expertsPerLayer"] * layout["expertStride"]
    for layer in layout["layers"]:
        if layer["experts"] and file_sizes.get("packed_experts/" + layer["file"]) != layer_size:
            raise LayoutInvalid("manifest.files.packed_experts/" + layer["file"], "missing or wrong layer size")


OFFSET_ROLES = ["gate", "gate_scales", "gate_biases", "up", "up_scales", "up_biases", "down", "down_scales",
                "down_biases", "gate_bias", "up_bias", "down_bias"]


def routed_expert_offsets(layout: dict, layer: int, additive_biases: bool = False) -> list:
    """Model.routedExpertOffsets, sources/Shrike/Runtime/Inference/ModelExpertIO.swift:69-94: offsets of
    expert 0's sub-tensors in the order of MoEExpertOffsets' fields, 0 for a role the blob lacks."""
    tensors = layout["layers"][layer]["experts"][0]["tensors"]
    if additive_biases:
        for role in ("gate_bias", "up_bias", "down_bias"):
            if role not in tensors:
                raise LayoutInvalid(f"layer {layer}", f"expert blob is missing {role}")
    return [tensors[r]["offset"] & U32_MAX if r in tensors else 0 for r in OFFSET_ROLES]


# ------------------------------------------------------------- parallel reader rules

def reader_claim_slot(slots) -> int:
    """shrike_expert_reader_claim_slot, sources/ShrikeKernelsC/expert_io.c:46-58: the oldest active slot
    with an unclaimed read. slots: (active, sequence, next_index, count)."""
    best = -1
    for i, (active, sequence, next_index, count) in enumerate(slots):
        if active and next_index < count and (best < 0 or sequence < slots[best][1]):
            best = i
    return best


def reader_free_slot(slots) -> int:
    """shrike_expert_reader_free_slot, expert_io.c:60-68."""
    for i, s in enumerate(slots):
        if not s[0]:
            return i
    return -1


def reader_cancel_slot(count, next_index, outstanding, first_errno, ecanceled):
    """shrike_expert_reader_cancel_slot, expert_io.c:70-80."""
    if next_index >= count:
        return count, next_index, outstanding, first_errno
    return count, count, outstanding - (count - next_index), first_errno or ecanceled


# ------------------------------------------------------------- routed tile loop of a streamed prefill chunk

class TileConfig:
    """PrefillRoutedTileSchedulerConfig, PrefillRoutedTileScheduler.swift:46-96."""

    def __init__(self, max_pending_depth=1, tile_experts=8, tiles_per_command_buffer=1, fetch_lookahead=0):
        self.max_pending_depth = max(1, max_pending_depth)
        self.tile_experts = max(1, min(16, tile_experts))
        self.tiles_per_command_buffer = max(1, min(16, tiles_per_command_buffer))
        self.fetch_lookahead = max(0, min(1, fetch_lookahead))

    def astuple(self):
        return (self.max_pending_depth, self.tile_experts, self.tiles_per_command_buffer, self.fetch_lookahead)

    @property
    def _batches(self):
        return self.max_pending_depth + 1

    def fits_slot_budget(self, slot_count, reserved_hits=0):
        if not (slot_count > 0 and reserved_hits >= 0):
            return False
        tiles = self._batches * self.tiles_per_command_buffer + self.fetch_lookahead
        return tiles * self.tile_experts + reserved_hits <= slot_count

    def fitting(self, slot_count, reserved_hits=0):
        if not (slot_count > reserved_hits and reserved_hits >= 0):
            return None
        available = slot_count - reserved_hits
        # Swift's `/` truncates toward zero; the numerator can be negative
        q = int((available - self.fetch_lookahead * self.tile_experts) / (self._batches * self.tile_experts))
        narrowed = TileConfig(self.max_pending_depth, self.tile_experts, max(1, min(self.tiles_per_command_buffer, q)),
                              self.fetch_lookahead)
        if narrowed.fits_slot_budget(slot_count, reserved_hits):
            return narrowed
        per_tile = available // (self._batches + self.fetch_lookahead)
        if per_tile <= 0:
            return None
        return TileConfig(self.max_pending_depth, min(self.tile_experts, per_tile), 1, self.fetch_lookahead)


def tile_decide(config, has_pending_tile, pending_assigned_slots, plan_available, pending_depth=None):
    """PrefillRoutedTileScheduler.decide, :104-122. Returns (decision, reason or avoiding slots)."""
    depth = max(0, pending_depth if pending_depth is not None else (1 if has_pending_tile else 0))
    if not has_pending_tile:
        return ("issueWithoutPending", None)
    if depth > config.max_pending_depth:
        return ("drainBeforeIssue", "maxPendingDepthReached")
    if not pending_assigned_slots:
        return ("drainBeforeIssue", "pendingTileHasNoAssignedSlots")
    if not plan_available:
        return ("drainBeforeIssue", "avoidingSlotPlanUnavailable")
    return ("prefetchNext", list(pending_assigned_slots))


def tile_batch_action(config, open_batch_tiles, open_batch_slots, next_plan_available, is_last_tile):
    """PrefillRoutedTileScheduler.batchAction, :139-155. Returns (commitBeforeAppend, closeReason or None)."""
    before = bool(open_batch_slots) and not next_plan_available
    after = (0 if before else max(0, open_batch_tiles)) + 1
    reason = "batchFull" if after >= config.tiles_per_command_buffer else "lastTile" if is_last_tile else None
    return before, reason


def tile_plans_lookahead(config, index, tile_count):
    return config.fetch_lookahead > 0 and index + 1 < tile_count


def tile_sequence(config, tile_count, driver):
    """PrefillRoutedTileSequencer.run, PrefillRoutedTileSequencer.swift:30-104, over a driver object with the
    protocol's members; an exception reaches abandon_begun_fetches and propagates."""
    def issue(tile, plan_available):
        decision, _ = tile_decide(config, driver.pending_depth > 0, driver.pending_assigned_slots, plan_available,
                                  driver.pending_depth)
        if decision == "drainBeforeIssue":
            if plan_available:
                driver.abandon_plan(tile)
            driver.drain_oldest_batch()
        driver.begin(tile)

    try:
        carried = None
        for tile in range(tile_count):
            is_last = tile == tile_count - 1
            carried_fetch = carried == tile
            carried = None
            plan_available = True if carried_fetch else driver.plan(tile, None)
            before, after = tile_batch_action(config, driver.open_batch_tiles, driver.open_batch_slots, plan_available, is_last)
            if before:
                driver.commit_open_batch()
            if not carried_fetch:
                issue(tile, plan_available)
            if tile_plans_lookahead(config, tile, tile_count):
                if driver.plan(tile + 1, tile):
                    driver.begin(tile + 1)
                    carried = tile + 1
            driver.encode(tile)
            if after is not None:
                driver.commit_open_batch()
            while driver.pending_depth + (1 if driver.open_batch_tiles > 0 else 0) > config.max_pending_depth:
                driver.drain_oldest_batch()
        driver.commit_open_batch()
        while driver.pending_depth > 0:
            driver.drain_oldest_batch()
    except BaseException:
        driver.abandon_begun_fetches()
        raise


# ------------------------------------------------------------------ load operations and the prefetch ring
# (sources/Shrike/Infrastructure/Streaming/ExpertLoadOperation.swift:15-153,
#  sources/Shrike/Runtime/Inference/ExpertPrefetchRing.swift:42-352). Pinned by the reference's own
# ExpertPrefetchRingTests vectors.

import threading as _threading
import time as _time

SUBMITTED, IN_FLIGHT, COMPLETED, FAILED = "submitted", "inFlight", "completed", "failed"


class LoadOperation:
    def __init__(self):
        self._cond = _threading.Condition()
        self.state, self.failure = SUBMITTED, None
        self.submitted_nanos, self.started_nanos, self.completed_nanos = _time.monotonic_ns(), 0, 0

    def mark_in_flight(self):
        with self._cond:
            assert self.state == SUBMITTED, "expert load operation started more than once"
            self.state, self.started_nanos = IN_FLIGHT, _time.monotonic_ns()

    def finish(self, failure=None):
        with self._cond:
            assert self.state in (SUBMITTED, IN_FLIGHT), "expert load operation completed more than once"
            self.completed_nanos = _time.monotonic_ns()
            self.state, self.failure = (FAILED, failure) if failure else (COMPLETED, None)
            self._cond.notify_all()

    def wait(self):
        with self._cond:
            while self.state in (SUBMITTED, IN_FLIGHT):
                self._cond.wait()
            if self.failure:
                raise RuntimeError(self.failure)

    def wait_until(self, deadline_nanos):
        with self._cond:
            while self.state in (SUBMITTED, IN_FLIGHT):
                now = _time.monotonic_ns()
                if now >= deadline_nanos:
                    return False
                self._cond.wait((deadline_nanos - now) / 1e9)
            return True


class ClaimRefused(Exception):
    pass


class _RingSlot:
    def __init__(self, cell):
        self.cell, self.layer, self.expert, self.operation, self.leased, self.demand = cell, -1, -1, None, False, False

    @property
    def in_flight(self):  # :60-71
        if self.expert < 0:
            return False
        return self.operation is None or self.operation.state in (SUBMITTED, IN_FLIGHT)


class PrefetchRing:
    ATTACH_SPIN_NANOS, IN_FLIGHT_BUDGET = 5_000_000, 1

    def __init__(self, cells, drop):
        if not cells or len(set(cells)) != len(cells):
            raise ValueError("invalid prefetch ring geometry")
        self.slots = [_RingSlot(c) for c in cells]
        self.drop, self.lock = drop, _threading.Lock()
        self.stats = dict(issued=0, adopted=0, reclaimed=0, deferred=0, overlapped=0, late=0, joined=0, refused=0,
                          failed=0, hook_failures=0, begin_nanos=0, leased_peak=0)

    @property
    def in_flight_count(self):
        with self.lock:
            return sum(1 for s in self.slots if s.in_flight)

    @property
    def leased_count(self):
        with self.lock:
            return sum(1 for s in self.slots if s.leased)

    def _reclaim(self, keeping):  # :333-351
        for s in self.slots:
            if s.leased or s.layer == keeping or s.operation is None:
                continue
            if s.operation.state == COMPLETED:
                self.drop(s.layer, s.expert, s.cell)
                self.stats["reclaimed"] += 1
                s.layer, s.expert, s.operation = -1, -1, None
            elif s.operation.state == FAILED:
                self.stats["failed"] += 1
                s.layer, s.expert, s.operation = -1, -1, None

    def begin(self, layer, experts, resident=(), deferred=False, issue=None):  # :108-164
        started = _time.monotonic_ns()
        try:
            self.lock.acquire()
            self._reclaim(layer)
            active = {s.expert for s in self.slots if s.layer == layer and s.expert >= 0}
            wanted = []
            for e in experts:
                if e not in resident and e not in active and e not in wanted:
                    wanted.append(e)
            free = [i for i, s in enumerate(self.slots) if s.expert < 0]
            budget = max(0, self.IN_FLIGHT_BUDGET - sum(1 for s in self.slots if s.in_flight))
            count = min(len(wanted), len(free), budget)
            self.stats["refused"] += len(wanted) - count
            if count == 0:
                self.lock.release()
                return
            chosen, chosen_experts = free[:count], wanted[:count]
            cells = [self.slots[i].cell for i in chosen]
            for i, e in zip(chosen, chosen_experts):
                self.slots[i].layer, self.slots[i].expert, self.slots[i].operation = layer, e, None
            self.lock.release()
            try:
                operation = issue(chosen_experts, cells)
            except BaseException as exc:
                with self.lock:
                    for i in chosen:
                        self.slots[i].layer, self.slots[i].expert, self.slots[i].operation = -1, -1, None
                    if isinstance(exc, ClaimRefused):
                        self.stats["refused"] += count
                        return
                raise
            with self.lock:
                for i in chosen:
                    self.slots[i].operation = operation
                self.stats["issued"] += count
                if deferred:
                    self.stats["deferred"] += 1
        finally:
            self.stats["begin_nanos"] += _time.monotonic_ns() - started

    def ready_cells(self, layer, experts, join_nanos=0):  # :171-212
        requested = set(experts)
        deadline = _time.monotonic_ns() + join_nanos if join_nanos > 0 else 0
        result, joined_ops, late_ops = {}, set(), set()
        self.lock.acquire()
        try:
            for s in self.slots:
                if s.layer != layer or s.expert not in requested:
                    continue
                if s.in_flight:
                    operation = self._attached(s)
                    if operation is None:
                        self.stats["late"] += 1
                        continue
                    self.lock.release()
                    joined = deadline > 0 and operation.wait_until(deadline)
                    if not joined:
                        try:
                            operation.wait()
                        except RuntimeError:
                            pass
                    self.lock.acquire()
                    (joined_ops if joined else late_ops).add(id(operation))
                    if s.layer != layer or s.expert not in requested:
                        continue
                if s.operation is None:
                    continue
                if id(s.operation) in joined_ops:
                    self.stats["joined"] += 1
                elif id(s.operation) in late_ops:
                    self.stats["late"] += 1
                if s.operation.state == COMPLETED:
                    result[s.expert] = s.cell
                    s.leased = True
            return result
        finally:
            self.lock.release()

    def _attached(self, s):  # :216-228
        if s.operation is not None:
            return s.operation
        layer, expert = s.layer, s.expert
        deadline = _time.monotonic_ns() + self.ATTACH_SPIN_NANOS
        while s.operation is None and _time.monotonic_ns() < deadline:
            self.lock.release()
            _time.sleep(50e-6)
            self.lock.acquire()
            if s.layer != layer or s.expert != expert:
                return None
        return s.operation

    def consume(self, layer, experts, freed_cells):  # :232-252
        with self.lock:
            for s in self.slots:
                if s.layer != layer or s.expert not in experts:
                    continue
                if s.expert in freed_cells:
                    s.cell = freed_cells[s.expert]
                else:
                    self.drop(layer, s.expert, s.cell)
                if not s.demand:
                    self.stats["adopted"] += 1
                s.layer, s.expert, s.operation, s.leased, s.demand = -1, -1, None, False, False

    def claim_demand(self, layer, experts):  # :257-282
        with self.lock:
            self._reclaim(layer)
            cells = {}
            for e in experts:
                own = next((s for s in self.slots if s.layer == layer and s.expert == e), None)
                if own is not None:
                    if own.leased or own.operation is None or own.operation.state != FAILED:
                        continue
                    self.stats["failed"] += 1
                    own.operation = None
                else:
                    own = next((s for s in self.slots if s.expert < 0), None)
                    if own is None:
                        break
                    own.layer, own.expert, own.operation = layer, e, None
                own.leased = own.demand = True
                cells[e] = own.cell
            self.stats["leased_peak"] = max(self.stats["leased_peak"], sum(1 for s in self.slots if s.leased))
            return cells

    def attach_demand(self, layer, experts, operation):
        with self.lock:
            for s in self.slots:
                if s.demand and s.layer == layer and s.expert in experts:
                    s.operation = operation

    def completion_nanos(self, layer, experts):
        with self.lock:
            return {s.expert: s.operation.completed_nanos for s in self.slots
                    if s.layer == layer and s.expert in experts and s.operation is not None and s.operation.state == COMPLETED}

    def unlease(self, layer, experts):
        with self.lock:
            for s in self.slots:
                if s.layer == layer and s.expert in experts:
                    s.leased = False

    def note_demand_submission(self):
        with self.lock:
            if any(s.in_flight for s in self.slots):
                self.stats["overlapped"] += 1

    def note_hook_failure(self):
        with self.lock:
            self.stats["hook_failures"] += 1
            return self.stats["hook_failures"] == 1

    @property
    def statistics(self):
        with self.lock:
            return dict(self.stats)
