// Measurement aids, not operators, and not part of libshrikehip: this file is built into a small library of its
// own (libshrikeprobe.so) that only the benchmark and its test load. An empty launch and a kernel that only
// reads a byte range of each listed pool cell: timed beside a real kernel on the same cells they give the two
// floors that bound it on this part, what a launch costs with nothing to do, and what moving the same bytes
// costs with no arithmetic and no dependent loads behind it.
#include "gemv_common.h"

namespace shrike {

// this library's own error text (libshrikehip's is not linked in)
static std::string g_probe_error;
void set_error(const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_probe_error = buf;
}
int hip_failed(hipError_t err, const char *what) {
    set_error("%s: %s", what, hipGetErrorString(err));
    return EIO;
}

__global__ __launch_bounds__(256) void k_probe_empty(uint32_t *sink) {
    if (sink == nullptr && threadIdx.x == 0xffffffffu) *sink = 0u;  // never true; keeps the argument live
}

// A wave reads kProbeLoads x 1 KiB (16 bytes a lane) of one cell's range.
constexpr uint32_t kProbeLoads = 4;

__global__ __launch_bounds__(256) void k_probe_read(PoolArg pool, uint64_t stride, const uint32_t *cells, uint32_t cell_count,
                                                    uint64_t byte_offset, uint32_t waves_per_cell, uint32_t loads_per_cell, uint32_t *sink) {
    warm_kernel_arguments(pool);
    const uint32_t lane = threadIdx.x & 63u, wave = blockIdx.x * 4u + wave_index();
    const uint32_t which = wave / waves_per_cell, part = wave % waves_per_cell;
    if (which >= cell_count) return;
    const uint4 *base = reinterpret_cast<const uint4 *>(cell_base_uniform(pool, cells[which], stride) + byte_offset);
    uint4 v[kProbeLoads];
#pragma unroll
    for (uint32_t i = 0; i < kProbeLoads; ++i) {
        const uint32_t load = part * kProbeLoads + i;
        v[i] = load < loads_per_cell ? base[size_t(load) * 64u + lane] : zero4();
    }
    uint32_t acc = 0;
#pragma unroll
    for (uint32_t i = 0; i < kProbeLoads; ++i) acc ^= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
    // the loads must not be optimised away; uniform int4 codes never fold to this word in practice,
    // and nothing reads the sink
    if (acc == 0x9E3779B9u) sink[0] = wave;
}

// One wave walks a chain of dependent loads: word i of the table holds the index of the next word. What a launch of
// `hops` hops costs beyond an empty launch, divided by hops, is one memory round trip as a kernel sees it.
__global__ __launch_bounds__(64) void k_probe_chase(const uint32_t *table, uint32_t hops, uint32_t start, uint32_t *sink) {
    uint32_t at = start;
    asm volatile("" : "+v"(at));  // a vector register: the hops are vector loads, as the kernels' row loads are
    for (uint32_t i = 0; i < hops; ++i) at = __builtin_nontemporal_load(table + at);
    if (at == 0xffffffffu) sink[0] = at;  // never true for a table of indices; keeps the chain live
}

// The device's constant-rate clock into a slot: a time stamp that sits in stream (or graph) order between other kernels.
__global__ void k_probe_timestamp(uint64_t *slot) {
    if (threadIdx.x == 0) *slot = wall_clock64();
}

// What a SIMD does with matrix and vector instructions side by side. Every wave runs `slots` slots; a slot is four
// v_mfma_f32_32x32x16_f16 (WHAT & 1) and thirty-two fp32 fused multiply-adds on eight independent chains (WHAT & 2),
// a matrix instruction followed by eight of the vector ones. One workgroup of 4 x waves_per_simd waves a compute unit.
typedef _Float16 probe_half8 __attribute__((ext_vector_type(8)));
typedef float probe_f32x16 __attribute__((ext_vector_type(16)));
template <int WHAT>
__global__ __launch_bounds__(1024) void k_probe_issue(uint32_t slots, const float *one, float *sink) {
    probe_half8 a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a[i] = _Float16(float(threadIdx.x & 7u) + float(i));
        b[i] = _Float16(0.5f * float(i));
    }
    probe_f32x16 c[4] = {{0}, {0}, {0}, {0}};
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = float(threadIdx.x + i);
    const float m = one[0];
    for (uint32_t it = 0; it < slots; ++it) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if (WHAT & 1) c[q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c[q], 0, 0, 0);
            if (WHAT & 2) {
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = fmaf(v[i], m, 1.0f);
            }
        }
    }
    float sum = 0.0f;
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int i = 0; i < 16; ++i) sum += c[q][i];
#pragma unroll
    for (int i = 0; i < 8; ++i) sum += v[i];
    if (sum == -1.0f) sink[0] = sum;  // sums of non-negative terms: never true; keeps the work live
}

}  // namespace shrike

using namespace shrike;

extern "C" {

const char *shrike_probe_last_error(void) { return g_probe_error.c_str(); }

int shrike_probe_empty_launch(void *stream, uint32_t workgroups, uint32_t *d_sink) {
    SHRIKE_REQUIRE(workgroups >= 1 && d_sink != nullptr, "probe: workgroups must be positive and the sink bound");
    hipLaunchKernelGGL(k_probe_empty, dim3(workgroups), dim3(256), 0, as_stream(stream), d_sink);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

int shrike_probe_read(void *stream, const shrike_pool_bases *pool, uint64_t pool_slot_stride, const uint32_t *d_cells,
                          uint32_t cell_count, uint64_t byte_offset, uint64_t bytes_per_cell, uint32_t *d_sink) {
    SHRIKE_REQUIRE(pool != nullptr && d_cells != nullptr && d_sink != nullptr, "probe: pool, cells and sink must be bound");
    SHRIKE_REQUIRE(cell_count >= 1 && bytes_per_cell >= 1024u, "probe: nothing to read");
    SHRIKE_REQUIRE(byte_offset % 16u == 0 && bytes_per_cell % 1024u == 0 && pool_slot_stride % 16u == 0,
                   "probe: the range must be 16-byte aligned and a multiple of 1 KiB long");
    SHRIKE_REQUIRE(byte_offset + bytes_per_cell <= pool_slot_stride, "probe: the range leaves the cell");
    PoolArg p;
    fill_pool(p, pool);
    const uint32_t loads = uint32_t(bytes_per_cell / 1024u);
    const uint32_t waves_per_cell = (loads + kProbeLoads - 1) / kProbeLoads;
    const uint32_t waves = waves_per_cell * cell_count;
    hipLaunchKernelGGL(k_probe_read, dim3((waves + 3) / 4), dim3(256), 0, as_stream(stream), p, pool_slot_stride, d_cells,
                       cell_count, byte_offset, waves_per_cell, loads, d_sink);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

// d_table: `words` 32-bit indices below `words` (the caller fills them; a stride of many cache lines between
// consecutive hops keeps every hop a miss). The chain starts at `start`.
int shrike_probe_dependent_loads(void *stream, const uint32_t *d_table, uint32_t words, uint32_t hops, uint32_t start, uint32_t *d_sink) {
    SHRIKE_REQUIRE(d_table != nullptr && d_sink != nullptr && words >= 1 && start < words, "probe: table, sink and a start inside the table");
    SHRIKE_REQUIRE(hops >= 1 && hops <= 4096u, "probe: 1...4096 hops");
    hipLaunchKernelGGL(k_probe_chase, dim3(1), dim3(64), 0, as_stream(stream), d_table, hops, start, d_sink);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}

// One thread stores wall_clock64() to *d_slot behind whatever the stream holds. The clock's rate in kHz comes from
// shrike_probe_wall_clock_khz (hipDeviceAttributeWallClockRate of the current device; 0 on failure).
int shrike_probe_timestamp(void *stream, uint64_t *d_slot) {
    SHRIKE_REQUIRE(d_slot != nullptr && reinterpret_cast<uintptr_t>(d_slot) % 8u == 0, "probe: the slot must be bound and 8-byte aligned");
    hipLaunchKernelGGL(k_probe_timestamp, dim3(1), dim3(64), 0, as_stream(stream), d_slot);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}
// what: 1 matrix instructions only, 2 vector only, 3 both. d_one: a float holding 1.0f (the multiplier, unknown to the
// compiler). One workgroup per compute unit of the current device.
int shrike_probe_issue(void *stream, uint32_t what, uint32_t waves_per_simd, uint32_t slots, const float *d_one, float *d_sink) {
    SHRIKE_REQUIRE(what >= 1 && what <= 3 && (waves_per_simd == 1 || waves_per_simd == 2 || waves_per_simd == 4), "probe: what 1...3, 1, 2 or 4 waves a SIMD");
    SHRIKE_REQUIRE(slots >= 1 && slots <= (1u << 20) && d_one != nullptr && d_sink != nullptr, "probe: 1...2^20 slots, multiplier and sink bound");
    int device = 0, units = 0;
    SHRIKE_HIP(hipGetDevice(&device));
    SHRIKE_HIP(hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device));
    const dim3 grid = dim3(static_cast<uint32_t>(units)), block = dim3(256u * waves_per_simd);
    if (what == 1) hipLaunchKernelGGL(k_probe_issue<1>, grid, block, 0, as_stream(stream), slots, d_one, d_sink);
    else if (what == 2) hipLaunchKernelGGL(k_probe_issue<2>, grid, block, 0, as_stream(stream), slots, d_one, d_sink);
    else hipLaunchKernelGGL(k_probe_issue<3>, grid, block, 0, as_stream(stream), slots, d_one, d_sink);
    SHRIKE_HIP(hipGetLastError());
    return 0;
}
int shrike_probe_wall_clock_khz(void) {
    int device = 0, khz = 0;
    if (hipGetDevice(&device) != hipSuccess || hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, device) != hipSuccess) return 0;
    return khz;
}

}  // extern "C"
