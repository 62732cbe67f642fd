// Host-side plumbing shared by the C-ABI translation units.
#pragma once

#include <hip/hip_runtime.h>

#include <cerrno>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "../../include/shrike_hip.h"

namespace shrike {

void set_error(const char *fmt, ...);
int hip_failed(hipError_t err, const char *what);  // records the error, returns EIO

#define SHRIKE_REQUIRE(cond, ...)            \
    do {                                     \
        if (!(cond)) {                       \
            ::shrike::set_error(__VA_ARGS__); \
            return EINVAL;                   \
        }                                    \
    } while (0)

#define SHRIKE_HIP(call)                                             \
    do {                                                             \
        hipError_t err__ = (call);                                   \
        if (err__ != hipSuccess) return ::shrike::hip_failed(err__, #call); \
    } while (0)

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

int check_moe_desc(const shrike_moe_desc *desc);  // runtime.hip
// decode_phase2.hip: looks up, for the current device, the address of the static scratch array of
// shrike_hip_moe_decode_layer_noalloc (once per device; later calls return at once)
int init_layer_scratch();

}  // namespace shrike

namespace shrike { struct RouteEntry; }

// MoE.swift:41-216: the handle keeps the shape it was made for, the router's fp32
// logits (routerLogits, MoE.swift:74) and the router's arrival counter.
constexpr unsigned kLayerBatchTokens = 16;  // tokens the fused layer takes in one call (a logit row and a route table each)
constexpr unsigned kCounterWords = 256;
constexpr unsigned kRouterTokenCounters = 128;  // first of the per-token arrival counters

struct shrike_hip_moe {
    shrike_moe_desc desc;
    int device;
    float *d_logits;        // fp32[kLayerBatchTokens][SHRIKE_MAX_ROUTER_EXPERTS]: this layer's logits (one row a token of a batch), the
                            // paired router's in the second row
    shrike::RouteEntry *d_route;  // [kLayerBatchTokens][SHRIKE_MAX_ROUTER_EXPERTS]: the fused layer's route tables, in d_logits' allocation
    uint32_t *d_counter;    // u32[kCounterWords], zero between launches: [0] the router's arrivals ([1] the paired router's), from
                            // [kRouterTokenCounters] one word a token of the several-token router
};
