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

// Streaming read of known size: every lane keeps eight 16-byte loads in flight, nothing is written unless the XOR of everything
// read is a value the caller chose (so the loads cannot be dropped). The machine's own read rate beside the published 8 TB/s.
__global__ __launch_bounds__(256) void calibration_read_kernel(const uint4 *src, uint64_t n16, uint32_t *sink, uint32_t magic) {
    const uint64_t nthr = (uint64_t)gridDim.x * blockDim.x, t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint4 acc = make_uint4(0u, 0u, 0u, 0u);
    uint64_t i = t;
    for (; i + 7u * nthr < n16; i += 8u * nthr) {
        uint4 v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] = src[i + (uint64_t)k * nthr];
#pragma unroll
        for (int k = 0; k < 8; ++k) { acc.x ^= v[k].x; acc.y ^= v[k].y; acc.z ^= v[k].z; acc.w ^= v[k].w; }
    }
    for (; i < n16; i += nthr) { const uint4 v = src[i]; acc.x ^= v.x; acc.y ^= v.y; acc.z ^= v.z; acc.w ^= v.w; }
    const uint32_t h = acc.x ^ acc.y ^ acc.z ^ acc.w;
    if (h == magic) sink[0] = h;
}

// Dense fp16 matrix-core loop: every wave issues `iters` rounds of eight independent v_mfma_f32_16x16x32_f16 on operands that stay in
// registers (no memory traffic at all); 16 * 16 * 32 * 2 flops each. The machine's own MFMA rate beside the published 2.5 PFLOP/s.
typedef _Float16 cal_half8 __attribute__((ext_vector_type(8)));
typedef float cal_float4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void calibration_mfma_kernel(uint32_t iters, float seed, float *sink) {
    cal_half8 a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) { a[i] = (_Float16)(seed * (float)(threadIdx.x % 7u + i)); b[i] = (_Float16)(seed * (float)(threadIdx.x % 5u + i)); }
    cal_float4 c[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) c[k] = cal_float4{0.0f, 0.0f, 0.0f, 0.0f};
    for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
        for (int k = 0; k < 8; ++k) c[k] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c[k], 0, 0, 0);
    }
    float tot = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; ++k) tot += c[k][0] + c[k][1] + c[k][2] + c[k][3];
    if (tot == 12345.678f) sink[0] = tot;
}
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

int redhip_calibration_read(const void *src_dev, uint64_t bytes, void *sink_dev, void *stream) {
    if (!src_dev || !sink_dev || !bytes || bytes % 16u) return 0;
    redhip::prof_set_stage(redhip::ST_OTHER);
    REDHIP_LAUNCH(redhip::calibration_read_kernel, dim3(4096), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<const uint4 *>(src_dev),
                  bytes / 16u, static_cast<uint32_t *>(sink_dev), 0x9e3779b9u);
    return hipGetLastError() == hipSuccess;
}

int redhip_calibration_mfma(uint32_t grid, uint32_t iters, void *sink_dev, uint64_t *flops, void *stream) {
    if (!grid || !iters || !sink_dev) return 0;
    redhip::prof_set_stage(redhip::ST_OTHER);
    REDHIP_LAUNCH(redhip::calibration_mfma_kernel, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream), iters, 0.0f, static_cast<float *>(sink_dev));
    if (flops) *flops = (uint64_t)grid * 4u * iters * 8u * (2ull * 16u * 16u * 32u);      // four waves per workgroup
    return hipGetLastError() == hipSuccess;
}

int redhip_calibration_empty(uint32_t grid, uint32_t block, void *stream) {
    if (!grid || !block || block > 1024u) return 0;
    redhip::prof_set_stage(redhip::ST_OTHER);
    REDHIP_LAUNCH(redhip::calibration_empty_kernel, dim3(grid), dim3(block), 0, static_cast<hipStream_t>(stream), 0);
    return hipGetLastError() == hipSuccess;
}

}  // extern "C"
