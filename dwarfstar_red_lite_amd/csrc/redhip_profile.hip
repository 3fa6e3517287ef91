// Per-stage kernel timing for benchmarks: the library-side counterpart of the reference's RL_ENGINE_PROFILE
// stage timers (native/redmetal_engine.m:1150-1164). Every launch made while profiling is on carries a start
// and a stop event that take the dispatch's own begin/end timestamps.
#include <mutex>
#include <vector>

#include "../../include/redhip_moe.h"
#include "redhip_internal.h"

namespace redhip {

namespace {
struct Rec { uint32_t stage; hipEvent_t a, b; };
struct Profiler {
    std::mutex mu;
    bool on = false;
    std::vector<Rec> recs;
    std::vector<hipEvent_t> pool;       // events are reused across begin/end rounds
    size_t next = 0;
};
Profiler g_prof;
thread_local uint32_t t_stage = ST_OTHER;
const char *const kStageNames[ST_COUNT] = {
    "other", "router_gemv", "route_select", "group_pairs", "gateup", "shared_gateup", "down_combine",
    "fused_experts", "batch_gateup", "batch_down", "batch_combine", "prefill_gateup", "prefill_down", "slice_sum"};
}  // namespace

void prof_set_stage(uint32_t stage) { t_stage = stage < ST_COUNT ? stage : ST_OTHER; }

BlockContext &block_context() {
    static thread_local BlockContext ctx;
    return ctx;
}

RouteGuard &route_guard() {
    static thread_local RouteGuard g;
    return g;
}

void prof_events(hipEvent_t *start, hipEvent_t *stop) {
    *start = *stop = nullptr;
    if (!g_prof.on) return;
    std::lock_guard<std::mutex> lk(g_prof.mu);
    if (!g_prof.on) return;
    while (g_prof.pool.size() < g_prof.next + 2u) {
        hipEvent_t e = nullptr;
        if (hipEventCreate(&e) != hipSuccess) return;
        g_prof.pool.push_back(e);
    }
    *start = g_prof.pool[g_prof.next++];
    *stop = g_prof.pool[g_prof.next++];
    g_prof.recs.push_back(Rec{t_stage, *start, *stop});
}

}  // namespace redhip

using namespace redhip;

namespace redhip {
// plain copy of known size: the yardstick for memory-traffic counters
__global__ __launch_bounds__(256) void calibration_copy_kernel(uint4 *dst, const uint4 *src, uint64_t n16) {
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (uint64_t)gridDim.x * blockDim.x) dst[i] = src[i];
}
// nothing at all: what a launch of a given grid costs by itself
__global__ void calibration_empty_kernel(int) {}
}  // namespace redhip

extern "C" {

uint32_t redhip_profile_stage_count(void) { return ST_COUNT; }
const char *redhip_profile_stage_name(uint32_t stage) { return stage < ST_COUNT ? kStageNames[stage] : ""; }

int redhip_profile_begin(void) {
    std::lock_guard<std::mutex> lk(g_prof.mu);
    g_prof.recs.clear();
    g_prof.next = 0;
    g_prof.on = true;
    return 1;
}

int redhip_profile_end(double *stage_ms, uint32_t *stage_launches, uint32_t n_stage) {
    if (hipDeviceSynchronize() != hipSuccess) return 0;
    std::lock_guard<std::mutex> lk(g_prof.mu);
    g_prof.on = false;
    for (uint32_t i = 0; i < n_stage; ++i) {
        if (stage_ms) stage_ms[i] = 0.0;
        if (stage_launches) stage_launches[i] = 0u;
    }
    int ok = 1;
    for (const Rec &r : g_prof.recs) {
        float ms = 0.0f;
        if (hipEventElapsedTime(&ms, r.a, r.b) != hipSuccess) { ok = 0; continue; }
        if (r.stage < n_stage) {
            if (stage_ms) stage_ms[r.stage] += (double)ms;
            if (stage_launches) stage_launches[r.stage] += 1u;
        }
    }
    g_prof.recs.clear();
    g_prof.next = 0;
    return ok;
}

int redhip_calibration_copy(void *dst_dev, const void *src_dev, uint64_t bytes, void *stream) {
    if (!dst_dev || !src_dev || !bytes || bytes % 16u) return 0;
    redhip::prof_set_stage(redhip::ST_OTHER);
    REDHIP_LAUNCH(redhip::calibration_copy_kernel, dim3(2048), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<uint4 *>(dst_dev),
                  static_cast<const uint4 *>(src_dev), bytes / 16u);
    return hipGetLastError() == hipSuccess;
}

int redhip_calibration_empty(uint32_t grid, uint32_t block, void *stream) {
    if (!grid || !block || block > 1024u) return 0;
    redhip::prof_set_stage(redhip::ST_OTHER);
    REDHIP_LAUNCH(redhip::calibration_empty_kernel, dim3(grid), dim3(block), 0, static_cast<hipStream_t>(stream), 0);
    return hipGetLastError() == hipSuccess;
}

}  // extern "C"
