// Handles, the HBM slot pool and the small pure functions of the C ABI.
#include "host_common.h"

#include "../../include/shrike_host.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

namespace shrike {

static thread_local std::string g_last_error;

void set_error(const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
}

int hip_failed(hipError_t err, const char *what) {
    set_error("%s failed: %s", what, hipGetErrorString(err));
    return EIO;
}

__global__ void k_store_u64(uint64_t *dst, uint64_t value) { *dst = value; }

// up to 32 residency words in one launch, in order (a later entry for the same expert wins)
struct StoreBatch {
    uint32_t count;
    uint32_t expert[32];
    uint64_t word[32];
};
__global__ void k_store_batch(uint64_t *table, StoreBatch b) {
    if (threadIdx.x != 0) return;
    for (uint32_t i = 0; i < b.count; ++i) table[b.expert[i]] = b.word[i];
}

}  // namespace shrike

using namespace shrike;

// ExpertCellArena.swift:16-133 + the residency table of PreadExpertStreamer.swift:283-352.
struct shrike_hip_pool {
    uint32_t cells, num_experts, cells_per_chunk, chunk_count;
    uint64_t stride;
    void *chunks[SHRIKE_POOL_MAX_CHUNKS];
    shrike_pool_bases bases;
    uint64_t *d_table;
    std::vector<uint64_t> shadow;  // host copy of the table, updated at publish
    bool owns_cells = true;        // false for a layer's table over another pool's cells
    // execute_plan's second copy queue: two host-to-device copies in flight fill the link better than one
    // (57 against 53 GB/s for 7 MB blobs from pinned memory); made at the first plan with two misses or more
    hipStream_t side_stream = nullptr;
    hipEvent_t side_fork = nullptr, side_join = nullptr;
};

namespace shrike {

// MoE.init's preconditions (MoE.swift:113-116 and the kernels' own ceilings); EINVAL with the cause recorded.
int check_moe_desc(const shrike_moe_desc *desc) {
    SHRIKE_REQUIRE(desc != nullptr, "desc is NULL");
    SHRIKE_REQUIRE(desc->routed_weight_bits == 4 || desc->routed_weight_bits == 8, "routedWeightBits=%u not in {4, 8}",
                   desc->routed_weight_bits);
    SHRIKE_REQUIRE(desc->router_weight_bits == 0 || desc->router_weight_bits == 4 || desc->router_weight_bits == 8,
                   "routerWeightBits=%u not in {0 (fp16), 4, 8}", desc->router_weight_bits);
    SHRIKE_REQUIRE(desc->top_k >= 1 && desc->top_k <= SHRIKE_MAX_TOP_K, "topK=%u not in 1...%u", desc->top_k, SHRIKE_MAX_TOP_K);
    SHRIKE_REQUIRE(desc->d != 0 && desc->d <= SHRIKE_MAX_HIDDEN && desc->d % SHRIKE_GROUP_SIZE == 0,
                   "d=%u must be a multiple of %u and at most %u", desc->d, SHRIKE_GROUP_SIZE, SHRIKE_MAX_HIDDEN);
    SHRIKE_REQUIRE(desc->f != 0 && desc->f % SHRIKE_GROUP_SIZE == 0, "f=%u must be a positive multiple of %u", desc->f,
                   SHRIKE_GROUP_SIZE);
    SHRIKE_REQUIRE(desc->num_experts >= desc->top_k && desc->num_experts <= SHRIKE_MAX_ROUTER_EXPERTS,
                   "numExperts=%u must be in topK...%u", desc->num_experts, SHRIKE_MAX_ROUTER_EXPERTS);
    SHRIKE_REQUIRE(desc->meta_dtype <= SHRIKE_META_F16 && desc->activation <= SHRIKE_ACT_CLAMPED_SWIGLU,
                   "metaDtype=%u or activation=%u is not a known value", desc->meta_dtype, desc->activation);
    return 0;
}

}  // namespace shrike

size_t shrike_expert_reader_stride_internal(const shrike_expert_reader *r);  // expert_io.cpp

extern "C" {

const char *shrike_hip_last_error(void) { return g_last_error.c_str(); }
const char *shrike_host_last_error(void) { return g_last_error.c_str(); }

int shrike_hip_init(int device) {
    int count = 0;
    SHRIKE_HIP(hipGetDeviceCount(&count));
    SHRIKE_REQUIRE(device >= 0 && device < count, "device %d of %d is not present", device, count);
    SHRIKE_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    SHRIKE_HIP(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        set_error("device %d is %s; this library carries gfx950 code only", device, prop.gcnArchName);
        return ENODEV;
    }
    return shrike::init_layer_scratch();  // the allocation-free layer's static scratch, found once per device
}

uint64_t shrike_expert_offsets_make(uint32_t d, uint32_t f, uint32_t bits, int additive_biases,
                                    shrike_expert_offsets *out) {
    if (!out || (bits != 4 && bits != 8) || d == 0 || f == 0 || d % SHRIKE_GROUP_SIZE || f % SHRIKE_GROUP_SIZE) {
        set_error("Offsets: d=%u and f=%u must be positive multiples of %u and bits=%u one of 4, 8", d, f,
                  SHRIKE_GROUP_SIZE, bits);
        return 0;
    }
    const uint64_t gate_codes = uint64_t(f) * d * bits / 8, gate_meta = uint64_t(f) * (d / SHRIKE_GROUP_SIZE) * 2;
    const uint64_t down_codes = uint64_t(d) * f * bits / 8, down_meta = uint64_t(d) * (f / SHRIKE_GROUP_SIZE) * 2;
    uint64_t at = 0;
    auto take = [&at](uint64_t size) { const uint64_t here = at; at += size; return uint32_t(here); };
    out->gate_w_off = take(gate_codes); out->gate_s_off = take(gate_meta); out->gate_b_off = take(gate_meta);
    out->up_w_off = take(gate_codes); out->up_s_off = take(gate_meta); out->up_b_off = take(gate_meta);
    out->down_w_off = take(down_codes); out->down_s_off = take(down_meta); out->down_b_off = take(down_meta);
    out->gate_ab_off = out->up_ab_off = out->down_ab_off = 0;
    if (additive_biases) {
        out->gate_ab_off = take(uint64_t(f) * 2); out->up_ab_off = take(uint64_t(f) * 2);
        out->down_ab_off = take(uint64_t(d) * 2);
    }
    return at;
}

// ------------------------------------------------------------------ budget

// RuntimeConfiguration.swift:111-129
int64_t shrike_parse_budget_bytes(const char *text) {
    if (!text) return -1;
    std::string raw(text);
    auto trim = [](std::string &s) {
        size_t a = 0, b = s.size();
        while (a < b && (s[a] == ' ' || s[a] == '\t')) ++a;  // Swift's .whitespaces: space and tab
        while (b > a && (s[b - 1] == ' ' || s[b - 1] == '\t')) --b;
        s = s.substr(a, b - a);
    };
    trim(raw);
    for (char &c : raw) c = char(toupper((unsigned char)c));
    if (raw.empty()) return -1;
    static const struct { const char *suffix; int64_t scale; } kMultipliers[] = {
        {"GIB", int64_t(1) << 30}, {"MIB", int64_t(1) << 20}, {"KIB", int64_t(1) << 10},
        {"GB", int64_t(1) << 30},  {"MB", int64_t(1) << 20},  {"KB", int64_t(1) << 10},
        {"G", int64_t(1) << 30},   {"M", int64_t(1) << 20},   {"K", int64_t(1) << 10},
    };
    for (const auto &m : kMultipliers) {
        const size_t n = strlen(m.suffix);
        if (raw.size() < n || raw.compare(raw.size() - n, n, m.suffix) != 0) continue;
        std::string number = raw.substr(0, raw.size() - n);
        trim(number);
        if (number.empty()) return -1;
        // Swift's Double(String): the whole string must parse; no leading/trailing blanks
        char *end = nullptr;
        errno = 0;
        const double value = strtod(number.c_str(), &end);
        if (end == number.c_str() || *end != '\0' || isspace((unsigned char)number[0])) return -1;
        if (!(value > 0)) return -1;
        const double bytes = value * double(m.scale);
        if (!std::isfinite(bytes) || bytes < 1 || !(bytes < 9223372036854775807.0)) return -1;
        return int64_t(bytes);
    }
    if (raw.empty()) return -1;
    size_t i = 0;
    if (raw[0] == '+' || raw[0] == '-') i = 1;
    if (i >= raw.size()) return -1;
    for (size_t j = i; j < raw.size(); ++j)
        if (raw[j] < '0' || raw[j] > '9') return -1;
    errno = 0;
    const long long plain = strtoll(raw.c_str(), nullptr, 10);
    if (errno == ERANGE || plain <= 0) return -1;
    return plain;
}

// RuntimeConfiguration.swift:77, :137-149
int32_t shrike_expert_cache_slots(uint64_t expert_stride_bytes, int32_t layers, int64_t budget_bytes) {
    static const int32_t kAllowed[] = {8, 16, 24, 32, 64, 96, 128, 160, 192, 224, 256};
    if (expert_stride_bytes == 0 || layers <= 0) return kAllowed[0];
    const double per_slot = double(expert_stride_bytes) * double(layers);
    const double wanted = double(budget_bytes) / per_slot;
    int32_t best = kAllowed[0];
    for (int32_t slots : kAllowed)  // Swift's min(by:) keeps the first of equal elements
        if (std::fabs(double(slots) - wanted) < std::fabs(double(best) - wanted)) best = slots;
    return best;
}

// -------------------------------------------------------------------- pool

shrike_hip_pool *shrike_hip_pool_create(uint32_t cells, uint64_t expert_stride, uint32_t num_experts,
                                        uint64_t chunk_bytes, int *out_errno) {
    auto fail = [&](int code) -> shrike_hip_pool * { if (out_errno) *out_errno = code; return nullptr; };
    if (cells == 0 || expert_stride == 0 || num_experts == 0) {
        set_error("invalid expert cell arena geometry: %u cells of %llu bytes for %u experts", cells,
                  (unsigned long long)expert_stride, num_experts);
        return fail(EINVAL);
    }
    // PreadExpertStreamer.swift:283-287: the slot stride is the expert stride rounded up to a page.
    const uint64_t stride = (expert_stride + SHRIKE_POOL_PAGE - 1) / SHRIKE_POOL_PAGE * SHRIKE_POOL_PAGE;
    // ExpertCellArena.swift:41-50
    const uint64_t limit = chunk_bytes ? chunk_bytes : ~uint64_t(0);
    uint64_t per_chunk = limit / stride;
    if (per_chunk < 1) per_chunk = 1;
    if (per_chunk > cells) per_chunk = cells;
    const uint32_t chunk_count = uint32_t((cells + per_chunk - 1) / per_chunk);
    if (chunk_count > SHRIKE_POOL_MAX_CHUNKS) {
        set_error("expert cell arena of %u cells needs %u chunks of %llu; the kernels address at most %u", cells,
                  chunk_count, (unsigned long long)per_chunk, SHRIKE_POOL_MAX_CHUNKS);
        return fail(EINVAL);
    }
    shrike_hip_pool *pool = new shrike_hip_pool();
    pool->cells = cells; pool->num_experts = num_experts; pool->stride = stride;
    pool->cells_per_chunk = uint32_t(per_chunk); pool->chunk_count = chunk_count;
    memset(pool->chunks, 0, sizeof(pool->chunks));
    pool->d_table = nullptr;
    for (uint32_t c = 0; c < chunk_count; ++c) {
        const uint64_t n = std::min<uint64_t>(per_chunk, cells - uint64_t(c) * per_chunk);
        if (hipMalloc(&pool->chunks[c], n * stride) != hipSuccess) {
            set_error("hipMalloc of %llu bytes for pool chunk %u failed", (unsigned long long)(n * stride), c);
            shrike_hip_pool_destroy(pool);
            return fail(ENOMEM);
        }
    }
    for (uint32_t i = 0; i < SHRIKE_POOL_MAX_CHUNKS; ++i)  // ExpertCellArena.swift:80-83
        pool->bases.base[i] = pool->chunks[i < chunk_count ? i : chunk_count - 1];
    pool->bases.cells_per_chunk = pool->cells_per_chunk;
    pool->shadow.assign(num_experts, uint64_t(SHRIKE_RESIDENCY_EMPTY) << 32 | SHRIKE_SLOT_SENTINEL);
    if (hipMalloc(reinterpret_cast<void **>(&pool->d_table), sizeof(uint64_t) * num_experts) != hipSuccess
        || hipMemcpy(pool->d_table, pool->shadow.data(), sizeof(uint64_t) * num_experts, hipMemcpyHostToDevice)
               != hipSuccess) {
        set_error("residency table allocation failed");
        shrike_hip_pool_destroy(pool);
        return fail(ENOMEM);
    }
    if (out_errno) *out_errno = 0;
    return pool;
}

shrike_hip_pool *shrike_hip_pool_create_layer_view(const shrike_hip_pool *arena, uint32_t num_experts, int *out_errno) {
    auto fail = [&](int code) -> shrike_hip_pool * { if (out_errno) *out_errno = code; return nullptr; };
    if (!arena || num_experts == 0) {
        set_error("a layer's residency table needs an arena and at least one expert");
        return fail(EINVAL);
    }
    shrike_hip_pool *pool = new shrike_hip_pool();
    pool->cells = arena->cells; pool->num_experts = num_experts; pool->stride = arena->stride;
    pool->cells_per_chunk = arena->cells_per_chunk; pool->chunk_count = arena->chunk_count;
    memcpy(pool->chunks, arena->chunks, sizeof(pool->chunks));
    pool->bases = arena->bases;
    pool->owns_cells = false;
    pool->d_table = nullptr;
    pool->shadow.assign(num_experts, uint64_t(SHRIKE_RESIDENCY_EMPTY) << 32 | SHRIKE_SLOT_SENTINEL);
    if (hipMalloc(reinterpret_cast<void **>(&pool->d_table), sizeof(uint64_t) * num_experts) != hipSuccess
        || hipMemcpy(pool->d_table, pool->shadow.data(), sizeof(uint64_t) * num_experts, hipMemcpyHostToDevice)
               != hipSuccess) {
        set_error("residency table allocation failed");
        shrike_hip_pool_destroy(pool);
        return fail(ENOMEM);
    }
    if (out_errno) *out_errno = 0;
    return pool;
}

void shrike_hip_pool_destroy(shrike_hip_pool *pool) {
    if (!pool) return;
    for (void *c : pool->chunks)
        if (c && pool->owns_cells) (void)hipFree(c);
    if (pool->d_table) (void)hipFree(pool->d_table);
    if (pool->side_stream) (void)hipStreamDestroy(pool->side_stream);
    if (pool->side_fork) (void)hipEventDestroy(pool->side_fork);
    if (pool->side_join) (void)hipEventDestroy(pool->side_join);
    delete pool;
}

uint64_t shrike_hip_pool_slot_stride(const shrike_hip_pool *pool) { return pool ? pool->stride : 0; }
uint32_t shrike_hip_pool_cell_count(const shrike_hip_pool *pool) { return pool ? pool->cells : 0; }

void *shrike_hip_pool_cell_ptr(const shrike_hip_pool *pool, uint32_t cell) {
    if (!pool || cell >= pool->cells) { set_error("expert cell out of range"); return nullptr; }
    return static_cast<uint8_t *>(pool->chunks[cell / pool->cells_per_chunk])
        + uint64_t(cell % pool->cells_per_chunk) * pool->stride;
}

const shrike_pool_bases *shrike_hip_pool_bases(const shrike_hip_pool *pool) { return pool ? &pool->bases : nullptr; }
void *shrike_hip_pool_residency_table(const shrike_hip_pool *pool) { return pool ? pool->d_table : nullptr; }

int shrike_hip_pool_upload_async(shrike_hip_pool *pool, uint32_t cell, const void *host_src, uint64_t bytes,
                                 void *stream) {
    SHRIKE_REQUIRE(pool && host_src, "pool or source is NULL");
    SHRIKE_REQUIRE(cell < pool->cells, "expert cell %u out of range (%u cells)", cell, pool->cells);
    SHRIKE_REQUIRE(bytes <= pool->stride, "%llu bytes do not fit a cell of %llu", (unsigned long long)bytes,
                   (unsigned long long)pool->stride);
    SHRIKE_HIP(hipMemcpyAsync(shrike_hip_pool_cell_ptr(pool, cell), host_src, bytes, hipMemcpyHostToDevice,
                              as_stream(stream)));
    return 0;
}

int shrike_hip_pool_fetch_experts(shrike_hip_pool *pool, void *stream, shrike_expert_reader *reader,
                                  const uint64_t *file_offsets, const uint32_t *cells, uint32_t count, uint64_t blob_bytes,
                                  void *pinned_staging, uint64_t staging_bytes) {
    SHRIKE_REQUIRE(pool && reader, "pool or reader is NULL");
    if (count == 0) return 0;
    SHRIKE_REQUIRE(file_offsets && cells && pinned_staging, "offsets, cells or staging is NULL");
    SHRIKE_REQUIRE(blob_bytes > 0 && blob_bytes <= pool->stride, "%llu bytes do not fit a cell of %llu",
                   (unsigned long long)blob_bytes, (unsigned long long)pool->stride);
    SHRIKE_REQUIRE(staging_bytes / blob_bytes >= 2, "the staging buffer must hold two blobs of %llu bytes",
                   (unsigned long long)blob_bytes);
    // the reader's workers write its own stride to every destination, and destinations sit blob_bytes apart
    SHRIKE_REQUIRE(shrike_expert_reader_stride_internal(reader) == blob_bytes,
                   "blob_bytes=%llu is not the stride the reader was created with (%llu)", (unsigned long long)blob_bytes,
                   (unsigned long long)shrike_expert_reader_stride_internal(reader));
    for (uint32_t i = 0; i < count; ++i)
        SHRIKE_REQUIRE(cells[i] < pool->cells, "expert cell %u out of range (%u cells)", cells[i], pool->cells);
    const uint32_t per_half = uint32_t(std::min<uint64_t>(staging_bytes / blob_bytes / 2, count));
    hipEvent_t copied[2] = {nullptr, nullptr};
    bool pending[2] = {false, false};
    int rc = 0;
    for (int h = 0; h < 2 && rc == 0; ++h)
        if (hipEventCreateWithFlags(&copied[h], hipEventDisableTiming) != hipSuccess) rc = hip_failed(hipGetLastError(), "hipEventCreate");
    std::vector<void *> destinations(per_half);
    uint32_t done = 0;
    for (int h = 0; done < count && rc == 0; h ^= 1) {
        const uint32_t n = std::min(per_half, count - done);
        uint8_t *half = static_cast<uint8_t *>(pinned_staging) + uint64_t(h) * per_half * blob_bytes;
        if (pending[h]) {  // the copies that last read this half
            if (hipEventSynchronize(copied[h]) != hipSuccess) { rc = hip_failed(hipGetLastError(), "hipEventSynchronize"); break; }
            pending[h] = false;
        }
        for (uint32_t i = 0; i < n; ++i) destinations[i] = half + uint64_t(i) * blob_bytes;
        rc = shrike_expert_reader_fetch_offsets(reader, file_offsets + done, destinations.data(), n);
        if (rc != 0) {
            set_error("expert read failed: %s", strerror(rc));
            break;
        }
        for (uint32_t i = 0; i < n && rc == 0; ++i)
            rc = shrike_hip_pool_upload_async(pool, cells[done + i], destinations[i], blob_bytes, stream);
        if (rc == 0 && hipEventRecord(copied[h], as_stream(stream)) != hipSuccess) rc = hip_failed(hipGetLastError(), "hipEventRecord");
        pending[h] = rc == 0;
        done += n;
    }
    // the staging buffer is the caller's again on return, also after a failure
    if (hipStreamSynchronize(as_stream(stream)) != hipSuccess && rc == 0) rc = hip_failed(hipGetLastError(), "hipStreamSynchronize");
    for (int h = 0; h < 2; ++h)
        if (copied[h]) (void)hipEventDestroy(copied[h]);
    return rc;
}

int shrike_hip_pool_table_publish(shrike_hip_pool *pool, uint32_t expert, uint32_t cell, uint32_t state,
                                  void *stream) {
    SHRIKE_REQUIRE(pool != nullptr, "pool is NULL");
    if (expert >= pool->num_experts) return 0;  // PreadExpertStreamer.swift:1144: out-of-range experts are ignored
    SHRIKE_REQUIRE(state <= SHRIKE_RESIDENCY_RESIDENT, "state %u is not a residency state", state);
    SHRIKE_REQUIRE(state == SHRIKE_RESIDENCY_EMPTY || cell < pool->cells, "cell %u out of range", cell);
    const uint32_t slot = state == SHRIKE_RESIDENCY_EMPTY ? SHRIKE_SLOT_SENTINEL : cell;
    const uint64_t word = uint64_t(state) << 32 | slot;
    pool->shadow[expert] = word;
    hipLaunchKernelGGL(k_store_u64, dim3(1), dim3(1), 0, as_stream(stream), pool->d_table + expert, word);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

int shrike_hip_pool_execute_plan(shrike_hip_pool *pool, shrike_slot_cache *cache, const shrike_expert_cache_plan *plan,
                                 const void *host_store, uint64_t store_expert_stride, uint64_t expert_bytes, void *stream,
                                 uint64_t elapsed_nanos) {
    SHRIKE_REQUIRE(pool && cache && plan, "execute plan: NULL argument");
    SHRIKE_REQUIRE(plan->miss_count == 0 || host_store, "execute plan: the plan has misses and no host store to read them from");
    SHRIKE_REQUIRE(expert_bytes <= pool->stride && expert_bytes <= store_expert_stride, "execute plan: expert bytes exceed a cell or the store's stride");
    // the reads (PreadExpertStreamer.swift:610-621): one host-to-device copy per miss into the cell the plan reserved.
    // With two misses or more every other copy goes to a second queue that starts behind what `stream` holds so far
    // and that `stream` waits for before anything else is put on it, so the caller sees one ordered stream.
    hipStream_t main_stream = as_stream(stream);
    bool two_queues = plan->miss_count >= 2;
    if (two_queues) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(main_stream, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            two_queues = false;  // a stream under capture keeps its copies to itself
        }
    }
    if (two_queues && pool->side_stream == nullptr) {
        // the queue and its two events are made together or not at all: on any failure the plan goes over one queue
        hipStream_t side = nullptr;
        hipEvent_t fork = nullptr, join = nullptr;
        // (another stream of this thread may be under a global-mode capture, which a stream creation would break:
        // the thread's capture mode is relaxed for the three calls)
        hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
        (void)hipThreadExchangeStreamCaptureMode(&mode);
        const bool made = hipStreamCreateWithFlags(&side, hipStreamNonBlocking) == hipSuccess
                          && hipEventCreateWithFlags(&fork, hipEventDisableTiming) == hipSuccess
                          && hipEventCreateWithFlags(&join, hipEventDisableTiming) == hipSuccess;
        (void)hipThreadExchangeStreamCaptureMode(&mode);
        if (made) {
            pool->side_stream = side; pool->side_fork = fork; pool->side_join = join;
        } else {
            (void)hipGetLastError();
            if (join) (void)hipEventDestroy(join);
            if (fork) (void)hipEventDestroy(fork);
            if (side) (void)hipStreamDestroy(side);
            two_queues = false;
        }
    }
    if (two_queues) {
        SHRIKE_HIP(hipEventRecord(pool->side_fork, main_stream));
        SHRIKE_HIP(hipStreamWaitEvent(pool->side_stream, pool->side_fork, 0));
    }
    // From here on the second queue may hold work: whatever ends the loop, `stream` waits for it before this call
    // returns, so that the caller's later work on `stream` is ordered behind every copy that was enqueued.
    int rc = 0;
    for (uint32_t m = 0; m < plan->miss_count && rc == 0; ++m) {
        const uint32_t i = plan->misses[m];
        const int32_t expert = plan->experts[i];
        if (expert < 0 || uint32_t(expert) >= pool->num_experts) {
            set_error("execute plan: expert %d out of range", expert);
            rc = EINVAL;
            break;
        }
        const uint64_t word = shrike_slot_cache_entry(cache, uint32_t(expert));
        const uint32_t cell = uint32_t(word);
        if (uint32_t(word >> 32) != SHRIKE_RESIDENCY_LOADING) {
            set_error("execute plan: expert %d is not loading (stale plan)", expert);
            rc = EINVAL;
        } else if (cell >= pool->cells) {
            set_error("execute plan: cell %u out of range", cell);
            rc = EINVAL;
        } else {
            const hipError_t err = hipMemcpyAsync(shrike_hip_pool_cell_ptr(pool, cell),
                                                  static_cast<const uint8_t *>(host_store) + uint64_t(expert) * store_expert_stride,
                                                  expert_bytes, hipMemcpyHostToDevice, two_queues && (m & 1u) ? pool->side_stream : main_stream);
            if (err != hipSuccess) rc = hip_failed(err, "execute plan: hipMemcpyAsync");
        }
    }
    if (two_queues) {
        hipError_t err = hipEventRecord(pool->side_join, pool->side_stream);
        if (err == hipSuccess) err = hipStreamWaitEvent(main_stream, pool->side_join, 0);
        if (err != hipSuccess) {
            // the join could not be enqueued: wait the second queue out on the host rather than leave it unordered
            (void)hipStreamSynchronize(pool->side_stream);
            if (rc == 0) rc = hip_failed(err, "execute plan: joining the second copy queue");
        }
    }
    if (rc != 0) return rc;
    // markPlanMissesResident, then every residency word that changed since the last drain goes to
    // the device table behind the copies on the same stream
    if (int rc = shrike_slot_cache_complete(cache, plan, elapsed_nanos, elapsed_nanos)) return rc;
    uint32_t experts[32];
    uint64_t words[32];
    for (;;) {
        const size_t n = shrike_slot_cache_drain_publications(cache, experts, words, 32);
        if (n == 0) break;
        StoreBatch b;
        b.count = 0;
        for (size_t i = 0; i < n; ++i) {
            if (experts[i] >= pool->num_experts) continue;
            pool->shadow[experts[i]] = words[i];
            b.expert[b.count] = experts[i];
            b.word[b.count] = words[i];
            ++b.count;
        }
        if (b.count) {
            hipLaunchKernelGGL(k_store_batch, dim3(1), dim3(64), 0, as_stream(stream), pool->d_table, b);
            SHRIKE_HIP(hipGetLastError());
        }
    }
    return 0;
}

uint64_t shrike_hip_pool_table_entry(const shrike_hip_pool *pool, uint32_t expert) {
    if (!pool || expert >= pool->num_experts) return uint64_t(SHRIKE_RESIDENCY_EMPTY) << 32 | SHRIKE_SLOT_SENTINEL;
    return pool->shadow[expert];
}

// --------------------------------------------------------------------- moe

// this layer's logits and the paired router's; the fused layer for a batch of tokens keeps a logit row and a route
// table per token
constexpr size_t kLogitsBytes = sizeof(float) * kLayerBatchTokens * SHRIKE_MAX_ROUTER_EXPERTS;
constexpr size_t kRouteBytes = 16u * kLayerBatchTokens * SHRIKE_MAX_ROUTER_EXPERTS;

shrike_hip_moe *shrike_hip_moe_create(const shrike_moe_desc *desc, int *out_errno) {
    auto fail = [&](int code) -> shrike_hip_moe * { if (out_errno) *out_errno = code; return nullptr; };
    if (int rc = shrike::check_moe_desc(desc)) return fail(rc);
    shrike_hip_moe *moe = new shrike_hip_moe();
    moe->desc = *desc;
    moe->d_logits = nullptr; moe->d_counter = nullptr;
    if (hipGetDevice(&moe->device) != hipSuccess
        || hipMalloc(reinterpret_cast<void **>(&moe->d_logits), kLogitsBytes + kRouteBytes) != hipSuccess
        || hipMalloc(reinterpret_cast<void **>(&moe->d_counter), sizeof(uint32_t) * kCounterWords) != hipSuccess
        || hipMemset(moe->d_counter, 0, sizeof(uint32_t) * kCounterWords) != hipSuccess
        || hipMemset(moe->d_logits, 0, kLogitsBytes + kRouteBytes) != hipSuccess) {
        set_error("device allocation for the MoE handle failed: %s", hipGetErrorString(hipGetLastError()));
        shrike_hip_moe_destroy(moe);
        return fail(ENOMEM);
    }
    moe->d_route = reinterpret_cast<shrike::RouteEntry *>(reinterpret_cast<unsigned char *>(moe->d_logits) + kLogitsBytes);
    if (out_errno) *out_errno = 0;
    return moe;
}

void shrike_hip_moe_destroy(shrike_hip_moe *moe) {
    if (!moe) return;
    if (moe->d_logits) (void)hipFree(moe->d_logits);
    if (moe->d_counter) (void)hipFree(moe->d_counter);
    delete moe;
}

}  // extern "C"

// ---------------------------------------------------------------- plumbing
// Device memory, streams, events and graphs for hosts that have no HIP binding of
// their own (the Python tests and benchmark). No counterpart in the reference: Metal
// buffers and command queues play this part there (MetalContext.swift).
extern "C" {

void *shrike_hip_malloc(uint64_t bytes) {
    void *p = nullptr;
    if (hipMalloc(&p, bytes ? bytes : 1) != hipSuccess) {
        set_error("hipMalloc(%llu) failed: %s", (unsigned long long)bytes, hipGetErrorString(hipGetLastError()));
        return nullptr;
    }
    return p;
}
int shrike_hip_free(void *p) { if (p) SHRIKE_HIP(hipFree(p)); return 0; }
void *shrike_hip_host_alloc(uint64_t bytes) {
    void *p = nullptr;
    if (hipHostMalloc(&p, bytes ? bytes : 1, hipHostMallocDefault) != hipSuccess) {
        set_error("hipHostMalloc(%llu) failed: %s", (unsigned long long)bytes, hipGetErrorString(hipGetLastError()));
        return nullptr;
    }
    return p;
}
int shrike_hip_host_free(void *p) { if (p) SHRIKE_HIP(hipHostFree(p)); return 0; }
int shrike_hip_memcpy_h2d(void *dst, const void *src, uint64_t bytes) {
    SHRIKE_HIP(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice)); return 0;
}
int shrike_hip_memcpy_d2h(void *dst, const void *src, uint64_t bytes) {
    SHRIKE_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost)); return 0;
}
int shrike_hip_memcpy_d2d(void *dst, const void *src, uint64_t bytes) {
    SHRIKE_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToDevice)); return 0;
}
int shrike_hip_memcpy_h2d_async(void *dst, const void *src, uint64_t bytes, void *stream) {
    SHRIKE_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(stream))); return 0;
}
int shrike_hip_memset(void *dst, int value, uint64_t bytes) { SHRIKE_HIP(hipMemset(dst, value, bytes)); return 0; }
int shrike_hip_device_synchronize(void) { SHRIKE_HIP(hipDeviceSynchronize()); return 0; }
int shrike_hip_mem_info(uint64_t *free_bytes, uint64_t *total_bytes) {
    size_t f = 0, t = 0;
    SHRIKE_HIP(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = t;
    return 0;
}

void *shrike_hip_stream_create(void) {
    hipStream_t s = nullptr;  // default priority only
    if (hipStreamCreateWithFlags(&s, hipStreamNonBlocking) != hipSuccess) {
        set_error("hipStreamCreate failed: %s", hipGetErrorString(hipGetLastError()));
        return nullptr;
    }
    return s;
}
int shrike_hip_stream_destroy(void *s) { if (s) SHRIKE_HIP(hipStreamDestroy(as_stream(s))); return 0; }
int shrike_hip_stream_synchronize(void *s) { SHRIKE_HIP(hipStreamSynchronize(as_stream(s))); return 0; }

void *shrike_hip_event_create(void) {
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) {
        set_error("hipEventCreate failed: %s", hipGetErrorString(hipGetLastError()));
        return nullptr;
    }
    return e;
}
int shrike_hip_event_destroy(void *e) { if (e) SHRIKE_HIP(hipEventDestroy(static_cast<hipEvent_t>(e))); return 0; }
int shrike_hip_event_record(void *e, void *stream) {
    SHRIKE_HIP(hipEventRecord(static_cast<hipEvent_t>(e), as_stream(stream))); return 0;
}
int shrike_hip_event_synchronize(void *e) { SHRIKE_HIP(hipEventSynchronize(static_cast<hipEvent_t>(e))); return 0; }
int shrike_hip_stream_wait_event(void *stream, void *e) {
    SHRIKE_HIP(hipStreamWaitEvent(as_stream(stream), static_cast<hipEvent_t>(e), 0)); return 0;
}
int shrike_hip_event_elapsed_ms(void *start, void *stop, float *ms) {
    SHRIKE_HIP(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop))); return 0;
}

int shrike_hip_graph_begin_capture(void *stream) {
    SHRIKE_REQUIRE(stream != nullptr, "graph capture needs an explicit stream");
    SHRIKE_HIP(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal)); return 0;
}
void *shrike_hip_graph_end_capture(void *stream) {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    if (hipStreamEndCapture(as_stream(stream), &graph) != hipSuccess || graph == nullptr) {
        set_error("hipStreamEndCapture failed: %s", hipGetErrorString(hipGetLastError()));
        return nullptr;
    }
    const hipError_t err = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (err != hipSuccess) { set_error("hipGraphInstantiate failed: %s", hipGetErrorString(err)); return nullptr; }
    return exec;
}
int shrike_hip_graph_launch(void *exec, void *stream) {
    SHRIKE_HIP(hipGraphLaunch(static_cast<hipGraphExec_t>(exec), as_stream(stream))); return 0;
}
int shrike_hip_graph_destroy(void *exec) {
    if (exec) SHRIKE_HIP(hipGraphExecDestroy(static_cast<hipGraphExec_t>(exec))); return 0;
}

}  // extern "C"
