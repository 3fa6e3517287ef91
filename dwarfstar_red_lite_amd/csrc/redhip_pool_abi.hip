// C-ABI front ends that keep the reference's call surface: the single-expert FFN pool (redmetal_ffn_*), the
// one-shot quantised GEMV (redmetal_quant_rows) and the router entry points. Host pointers in, host pointers
// out, synchronous; the arithmetic runs in the gfx950 kernels of redhip_kernels.hip.
#include <errno.h>
#include <fcntl.h>
#include <limits.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>
#include <sys/stat.h>
#include <time.h>
#include <unistd.h>

#include <mutex>
#include <vector>

#include "../../include/redmetal_ffn.h"
#include "../../include/redmetal_quant.h"
#include "../../include/redmetal_router.h"
#include "redhip_host_util.h"
#include "redhip_internal.h"

using namespace redhip;

namespace {

thread_local char g_ffn_error[512];
thread_local char g_quant_error[512];

#define FFN_ERR(...) set_err(g_ffn_error, sizeof(g_ffn_error), __VA_ARGS__)
#define QUANT_ERR(...) set_err(g_quant_error, sizeof(g_quant_error), __VA_ARGS__)

struct FfnPool {
    int fd = -1;
    uint64_t file_size = 0, slot_bytes = 0, budget = 0, allocated = 0;
    uint32_t capacity = 0, slots_per_slab = 0;
    std::vector<uint8_t *> slabs;                 // device memory, created on first use of a slot in the slab
    std::vector<uint32_t> inflight;
    std::vector<uint64_t> loaded_bytes;           // per slot: payload bytes of the last successful load_expert (0: never loaded)
    std::mutex mu;                                // counters, slab creation, in-flight marks, loaded_bytes
    std::mutex exec_mu;                           // the scratch below serves one execute at a time
    DevBuf scratch;
    uint64_t bytes_read = 0, read_calls = 0;
    double read_ms = 0.0;
    std::vector<int8_t> iq2_xs, iq1_m;            // the caller's codebooks (the reference keeps them in two device buffers per pool)

    uint8_t *slot_base(uint32_t slot) {           // nullptr + message on failure
        if (slot >= capacity) { FFN_ERR("FFN slot %u exceeds capacity %u", slot, capacity); return nullptr; }
        const uint32_t slab = slot / slots_per_slab;
        std::lock_guard<std::mutex> lk(mu);
        while (slabs.size() <= slab) {
            const uint32_t idx = (uint32_t)slabs.size();
            const uint32_t first = idx * slots_per_slab;
            const uint32_t n = capacity - first < slots_per_slab ? capacity - first : slots_per_slab;
            void *p = nullptr;
            const hipError_t e = hipMalloc(&p, (size_t)n * slot_bytes);
            if (e != hipSuccess) { FFN_ERR("failed to allocate FFN slab %u (%llu bytes): %s", idx, (unsigned long long)n * slot_bytes, hipGetErrorString(e)); return nullptr; }
            slabs.push_back(static_cast<uint8_t *>(p));
            allocated += (uint64_t)n * slot_bytes;
        }
        return slabs[slab] + (uint64_t)(slot % slots_per_slab) * slot_bytes;
    }
    uint8_t *slot_base_existing(uint32_t slot) {  // nullptr when the slot's slab has not been created yet; allocates nothing
        if (slot >= capacity) return nullptr;
        std::lock_guard<std::mutex> lk(mu);
        const uint32_t slab = slot / slots_per_slab;
        return slab < slabs.size() ? slabs[slab] + (uint64_t)(slot % slots_per_slab) * slot_bytes : nullptr;
    }
    void mark(uint32_t slot, int delta) {
        std::lock_guard<std::mutex> lk(mu);
        if (delta > 0) inflight[slot] += (uint32_t)delta;
        else if (inflight[slot]) inflight[slot] -= 1u;
    }
};

FfnPool *pool_of(redmetal_ffn_pool_t h) { return static_cast<FfnPool *>(h); }

// ---- scratch of redmetal_ffn_pool_execute_expert_noalloc: the SwiGLU activations between its two launches live in one array that is
// part of the library's device image, so the call never allocates. Every GPU holds its own copy at its own address; the address is
// looked up once per device (with that device current) and host code uses only that pointer, never the array's name.
constexpr uint32_t kNoAllocMaxFfn = 16384u;                                  // 64 KB per GPU, held until the process ends
static __device__ __align__(256) float scratch[kNoAllocMaxFfn];
constexpr int kMaxDevices = 64;
float *g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mu;

// the current device's copy of `scratch`; nullptr + message on failure
float *scratch_of_current_device(char *err, size_t cap) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) { set_err(err, cap, "no usable current HIP device for the static scratch (device %d): %s", dev, hipGetErrorString(e)); return nullptr; }
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) { set_err(err, cap, "hipGetSymbolAddress of the static scratch failed on device %d: %s", dev, hipGetErrorString(e)); return nullptr; }
        g_scratch_ptr[dev] = static_cast<float *>(p);
    }
    return g_scratch_ptr[dev];
}

}  // namespace

extern "C" {

// ------------------------------------------------------------------ redmetal_ffn

uint32_t redmetal_ffn_abi_version(void) { return 1u; }
const char *redmetal_ffn_last_error(void) { return g_ffn_error[0] ? g_ffn_error : "unknown Red Metal FFN error"; }

redmetal_ffn_pool_t redmetal_ffn_pool_create(const char *model_path, uint64_t budget_bytes, uint64_t slot_bytes,
        uint32_t slots_per_slab, const int8_t *iq2_xs_grid, uint32_t iq2_xs_grid_count,
        const int8_t *iq1_m_grid, uint32_t iq1_m_grid_count) {
    g_ffn_error[0] = '\0';
    if (!model_path || !model_path[0] || !budget_bytes || !slot_bytes || !iq2_xs_grid || !iq1_m_grid ||
        iq2_xs_grid_count != 512u * 8u || iq1_m_grid_count != 2048u * 8u) {
        FFN_ERR("invalid Red Metal FFN pool arguments");
        return nullptr;
    }
    if (slot_bytes > UINT64_MAX - 4095u) { FFN_ERR("FFN slot size overflow"); return nullptr; }
    const uint64_t aligned = (slot_bytes + 4095u) & ~4095ull;
    if (!aligned || aligned > budget_bytes) { FFN_ERR("FFN cache budget cannot fit one aligned expert slot"); return nullptr; }
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev < 1) { FFN_ERR("no HIP device available"); return nullptr; }
    if (!scratch_of_current_device(g_ffn_error, sizeof(g_ffn_error))) return nullptr;      // set-up of the entry point that allocates nothing
    FfnPool *p = new FfnPool();
    p->iq2_xs.assign(iq2_xs_grid, iq2_xs_grid + iq2_xs_grid_count);      // uploaded when an IQ2_XS / IQ1_M expert is executed
    p->iq1_m.assign(iq1_m_grid, iq1_m_grid + iq1_m_grid_count);
    p->slot_bytes = aligned;
    p->budget = budget_bytes;
    const uint64_t cap64 = budget_bytes / aligned;
    p->capacity = cap64 > 0xffffffffull ? 0xffffffffu : (uint32_t)cap64;
    p->slots_per_slab = slots_per_slab ? slots_per_slab : 64u;
    if (p->slots_per_slab > p->capacity) p->slots_per_slab = p->capacity;
    p->fd = open(model_path, O_RDONLY);
    if (p->fd < 0) { FFN_ERR("open(%s) failed: %s", model_path, strerror(errno)); delete p; return nullptr; }
    struct stat st;
    if (fstat(p->fd, &st) != 0 || st.st_size <= 0) {
        FFN_ERR("failed to stat model file: %s", strerror(errno));
        close(p->fd);
        delete p;
        return nullptr;
    }
    p->file_size = (uint64_t)st.st_size;
    p->inflight.assign(p->capacity, 0u);
    p->loaded_bytes.assign(p->capacity, 0u);
    return p;
}

void redmetal_ffn_pool_destroy(redmetal_ffn_pool_t handle) {
    FfnPool *p = pool_of(handle);
    if (!p) return;
    (void)hipDeviceSynchronize();
    for (uint8_t *s : p->slabs) (void)hipFree(s);
    if (p->fd >= 0) close(p->fd);
    forget_caller_grids(p);
    delete p;
}

uint32_t redmetal_ffn_pool_capacity(redmetal_ffn_pool_t h) { return h ? pool_of(h)->capacity : 0u; }
uint32_t redmetal_ffn_pool_slab_count(redmetal_ffn_pool_t h) {
    if (!h) return 0u;
    std::lock_guard<std::mutex> lk(pool_of(h)->mu);
    return (uint32_t)pool_of(h)->slabs.size();
}
uint64_t redmetal_ffn_pool_allocated_bytes(redmetal_ffn_pool_t h) {
    if (!h) return 0u;
    std::lock_guard<std::mutex> lk(pool_of(h)->mu);
    return pool_of(h)->allocated;
}
uint64_t redmetal_ffn_pool_bytes_read(redmetal_ffn_pool_t h) {
    if (!h) return 0u;
    std::lock_guard<std::mutex> lk(pool_of(h)->mu);
    return pool_of(h)->bytes_read;
}
uint64_t redmetal_ffn_pool_read_calls(redmetal_ffn_pool_t h) {
    if (!h) return 0u;
    std::lock_guard<std::mutex> lk(pool_of(h)->mu);
    return pool_of(h)->read_calls;
}
double redmetal_ffn_pool_read_ms(redmetal_ffn_pool_t h) {
    if (!h) return 0.0;
    std::lock_guard<std::mutex> lk(pool_of(h)->mu);
    return pool_of(h)->read_ms;
}
int redmetal_ffn_pool_slot_inflight(redmetal_ffn_pool_t h, uint32_t slot_id) {
    FfnPool *p = pool_of(h);
    if (!p || slot_id >= p->capacity) return 0;
    std::lock_guard<std::mutex> lk(p->mu);
    return p->inflight[slot_id] != 0u;
}

int redmetal_ffn_pool_load_expert(redmetal_ffn_pool_t h, uint32_t slot_id,
        uint64_t gate_file_offset, uint64_t gate_bytes, uint64_t up_file_offset, uint64_t up_bytes,
        uint64_t down_file_offset, uint64_t down_bytes, uint64_t *bytes_read, double *elapsed_ms) {
    FfnPool *p = pool_of(h);
    if (!p || slot_id >= p->capacity) return 0;
    if (redmetal_ffn_pool_slot_inflight(h, slot_id)) { FFN_ERR("refusing to overwrite in-flight FFN slot %u", slot_id); return 0; }
    if (sizes_overflow(gate_bytes, up_bytes, down_bytes)) { FFN_ERR("FFN expert payload size overflow"); return 0; }
    const uint64_t payload = gate_bytes + up_bytes + down_bytes;
    if (payload > p->slot_bytes) { FFN_ERR("FFN expert payload exceeds slot size"); return 0; }
    uint8_t *base = p->slot_base(slot_id);
    if (!base) return 0;
    std::vector<uint8_t> host((size_t)payload);
    uint64_t local_bytes = 0, local_calls = 0;
    const double t0 = now_ms();
    const bool ok =
        pread_range(p->fd, p->file_size, gate_file_offset, gate_bytes, host.data(), &local_bytes, &local_calls, g_ffn_error, sizeof(g_ffn_error)) &&
        pread_range(p->fd, p->file_size, up_file_offset, up_bytes, host.data() + gate_bytes, &local_bytes, &local_calls, g_ffn_error, sizeof(g_ffn_error)) &&
        pread_range(p->fd, p->file_size, down_file_offset, down_bytes, host.data() + gate_bytes + up_bytes, &local_bytes, &local_calls, g_ffn_error, sizeof(g_ffn_error));
    if (!ok) return 0;
    if (payload) {
        const hipError_t e = hipMemcpy(base, host.data(), (size_t)payload, hipMemcpyHostToDevice);
        if (e != hipSuccess) { FFN_ERR("FFN slot upload failed: %s", hipGetErrorString(e)); return 0; }
    }
    const double ms = now_ms() - t0;
    {
        std::lock_guard<std::mutex> lk(p->mu);
        p->bytes_read += local_bytes;
        p->read_calls += local_calls;
        p->read_ms += ms;
        p->loaded_bytes[slot_id] = payload;
    }
    if (bytes_read) *bytes_read = local_bytes;
    if (elapsed_ms) *elapsed_ms = ms;
    return 1;
}

int redmetal_ffn_pool_slot_addresses(redmetal_ffn_pool_t h, uint32_t slot_id, uint64_t gate_bytes, uint64_t up_bytes,
        uint64_t down_bytes, uint64_t *gate_address, uint64_t *up_address, uint64_t *down_address) {
    FfnPool *p = pool_of(h);
    if (!p || slot_id >= p->capacity) return 0;
    if (sizes_overflow(gate_bytes, up_bytes, down_bytes) || gate_bytes + up_bytes + down_bytes > p->slot_bytes) return 0;
    uint8_t *base = p->slot_base(slot_id);
    if (!base) return 0;
    const uint64_t a = (uint64_t)(uintptr_t)base;
    if (gate_address) *gate_address = a;
    if (up_address) *up_address = a + gate_bytes;
    if (down_address) *down_address = a + gate_bytes + up_bytes;
    return 1;
}

int redmetal_ffn_pool_execute_expert(redmetal_ffn_pool_t h, uint32_t slot_id, uint32_t ggml_type,
        uint64_t gate_bytes, uint64_t up_bytes, uint64_t down_bytes, uint32_t hidden_size, uint32_t ffn_size,
        uint32_t output_row_start, uint32_t output_row_count, const float *input, uint32_t input_count,
        float *output, uint32_t output_count, double *elapsed_ms) {
    FfnPool *p = pool_of(h);
    if (!p || !input || !output || slot_id >= p->capacity) return 0;
    const uint32_t gu = word_gate_up(ggml_type), dn = word_down(ggml_type);
    if (!pool_quant_supported(gu) || !pool_quant_supported(dn) || (ggml_type >> 16)) {
        FFN_ERR("unsupported FFN GGML type word 0x%x (supported: IQ2_XS 17, IQ1_M 29, IQ2_XXS 16, IQ3_S 21, Q6_K 14)", ggml_type);
        return 0;
    }
    if (!hidden_size || hidden_size % 256u || !ffn_size || ffn_size % 256u || input_count != hidden_size ||
        !output_row_count || output_row_start >= hidden_size || output_row_count > hidden_size - output_row_start ||
        output_count < output_row_count) {
        FFN_ERR("invalid FFN dimensions hidden=%u ffn=%u start=%u count=%u", hidden_size, ffn_size, output_row_start, output_row_count);
        return 0;
    }
    const uint64_t expect_gate = (uint64_t)ffn_size * pool_row_bytes(gu, hidden_size);
    const uint64_t expect_down = (uint64_t)hidden_size * pool_row_bytes(dn, ffn_size);
    if (gate_bytes != expect_gate || up_bytes != expect_gate || down_bytes != expect_down) {
        FFN_ERR("FFN matrix byte mismatch gate=%llu/%llu up=%llu/%llu down=%llu/%llu", (unsigned long long)gate_bytes,
                (unsigned long long)expect_gate, (unsigned long long)up_bytes, (unsigned long long)expect_gate,
                (unsigned long long)down_bytes, (unsigned long long)expect_down);
        return 0;
    }
    if (sizes_overflow(gate_bytes, up_bytes, down_bytes) || gate_bytes + up_bytes + down_bytes > p->slot_bytes) {
        FFN_ERR("FFN resident expert exceeds slot bounds");
        return 0;
    }
    uint8_t *base = p->slot_base(slot_id);
    if (!base) return 0;

    std::lock_guard<std::mutex> exec(p->exec_mu);
    const size_t n_x = hidden_size, n_act = ffn_size, n_out = output_row_count;
    if (!p->scratch.reserve((n_x + n_act + n_out) * sizeof(float))) { FFN_ERR("failed to allocate FFN activation buffers"); return 0; }
    float *dx = static_cast<float *>(p->scratch.p), *dact = dx + n_x, *dout = dact + n_act;
    hipError_t e = hipMemcpy(dx, input, n_x * sizeof(float), hipMemcpyHostToDevice);
    if (e != hipSuccess) { FFN_ERR("FFN input upload failed: %s", hipGetErrorString(e)); return 0; }
    if (gu == T_IQ2_XS || gu == T_IQ1_M || dn == T_IQ2_XS || dn == T_IQ1_M) {      // this pool's codebooks on the device (free when they already are)
        e = set_caller_grids(p->iq2_xs.data(), p->iq1_m.data(), p);
        if (e == hipErrorContextAlreadyInUse) { FFN_ERR("%s", kCodebookConflict); return 0; }
        if (e != hipSuccess) { FFN_ERR("failed to upload the IQ2_XS / IQ1_M codebooks: %s", hipGetErrorString(e)); return 0; }
    }
    p->mark(slot_id, 1);
    const double t0 = now_ms();
    ExpertSet ex{base, 0, gate_bytes, up_bytes, gu, dn};
    e = launch_moe_gateup(ex, nullptr, 1u, hidden_size, ffn_size, dx, dact, nullptr);
    if (e == hipSuccess) e = launch_gemv_rows(dn, base + gate_bytes + up_bytes, ffn_size, output_row_start, output_row_count, dact, dout, nullptr);
    if (e == hipSuccess) e = hipStreamSynchronize(nullptr);
    const double ms = now_ms() - t0;
    p->mark(slot_id, -1);
    if (e != hipSuccess) { FFN_ERR("FFN HIP command failed: %s", hipGetErrorString(e)); return 0; }
    e = hipMemcpy(output, dout, n_out * sizeof(float), hipMemcpyDeviceToHost);
    if (e != hipSuccess) { FFN_ERR("FFN output download failed: %s", hipGetErrorString(e)); return 0; }
    if (elapsed_ms) *elapsed_ms = ms;
    return 1;
}

int redmetal_ffn_pool_execute_expert_noalloc(redmetal_ffn_pool_t h, uint32_t slot_id, uint32_t ggml_type,
        uint64_t gate_bytes, uint64_t up_bytes, uint64_t down_bytes, uint32_t hidden_size, uint32_t ffn_size,
        uint32_t output_row_start, uint32_t output_row_count, const float *input_dev, uint32_t input_count,
        float *output_dev, uint32_t output_count, void *stream) {
    FfnPool *p = pool_of(h);
    if (!p || !input_dev || !output_dev || slot_id >= p->capacity) { FFN_ERR("invalid arguments of the non-allocating FFN call"); return 0; }
    const uint32_t gu = word_gate_up(ggml_type), dn = word_down(ggml_type);
    if (!pool_quant_supported(gu) || !pool_quant_supported(dn) || (ggml_type >> 16)) {
        FFN_ERR("unsupported FFN GGML type word 0x%x (supported: IQ2_XS 17, IQ1_M 29, IQ2_XXS 16, IQ3_S 21, Q6_K 14)", ggml_type);
        return 0;
    }
    if (ffn_size > kNoAllocMaxFfn) {
        FFN_ERR("ffn %u exceeds the static scratch of the non-allocating FFN call (at most %u activations)", ffn_size, kNoAllocMaxFfn);
        return 0;
    }
    if (!hidden_size || hidden_size % 256u || !ffn_size || ffn_size % 256u || input_count != hidden_size ||
        !output_row_count || output_row_start >= hidden_size || output_row_count > hidden_size - output_row_start ||
        output_count < output_row_count) {
        FFN_ERR("invalid FFN dimensions hidden=%u ffn=%u start=%u count=%u", hidden_size, ffn_size, output_row_start, output_row_count);
        return 0;
    }
    const uint64_t expect_gate = (uint64_t)ffn_size * pool_row_bytes(gu, hidden_size);
    const uint64_t expect_down = (uint64_t)hidden_size * pool_row_bytes(dn, ffn_size);
    if (gate_bytes != expect_gate || up_bytes != expect_gate || down_bytes != expect_down) {
        FFN_ERR("FFN matrix byte mismatch gate=%llu/%llu up=%llu/%llu down=%llu/%llu", (unsigned long long)gate_bytes,
                (unsigned long long)expect_gate, (unsigned long long)up_bytes, (unsigned long long)expect_gate,
                (unsigned long long)down_bytes, (unsigned long long)expect_down);
        return 0;
    }
    if (sizes_overflow(gate_bytes, up_bytes, down_bytes) || gate_bytes + up_bytes + down_bytes > p->slot_bytes) {
        FFN_ERR("FFN resident expert exceeds slot bounds");
        return 0;
    }
    uint8_t *base = p->slot_base_existing(slot_id);
    uint64_t loaded = 0;
    if (base) { std::lock_guard<std::mutex> lk(p->mu); loaded = p->loaded_bytes[slot_id]; }
    if (!base || !loaded) { FFN_ERR("FFN slot %u holds no expert yet: load it before the non-allocating call", slot_id); return 0; }
    if (gate_bytes + up_bytes + down_bytes > loaded) {
        FFN_ERR("FFN slot %u holds %llu bytes, the call names %llu", slot_id, (unsigned long long)loaded, (unsigned long long)(gate_bytes + up_bytes + down_bytes));
        return 0;
    }
    if ((gu == T_IQ2_XS || gu == T_IQ1_M || dn == T_IQ2_XS || dn == T_IQ1_M) && !caller_grids_bound(p)) {
        FFN_ERR("the pool's IQ2_XS / IQ1_M codebooks are not on the device yet: run redmetal_ffn_pool_execute_expert on such an expert once first");
        return 0;
    }
    float *act = scratch_of_current_device(g_ffn_error, sizeof(g_ffn_error));      // looked up at pool_create; a table read here
    if (!act) return 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // gate/up + SwiGLU writes act[0 .. ffn), the down rows read exactly that range: nothing in the scratch has to start at zero
    const ExpertSet ex{base, 0, gate_bytes, up_bytes, gu, dn};
    hipError_t e = launch_moe_gateup(ex, nullptr, 1u, hidden_size, ffn_size, input_dev, act, s);
    if (e == hipSuccess) e = launch_gemv_rows(dn, base + gate_bytes + up_bytes, ffn_size, output_row_start, output_row_count, act, output_dev, s);
    if (e != hipSuccess) { FFN_ERR("FFN HIP command failed: %s", hipGetErrorString(e)); return 0; }
    return 1;
}

// ------------------------------------------------------------------ redmetal_quant

uint32_t redmetal_quant_abi_version(void) { return 1u; }
const char *redmetal_quant_last_error(void) { return g_quant_error[0] ? g_quant_error : "unknown Red Metal quant error"; }

int redmetal_quant_rows(const char *model_path, uint64_t matrix_file_offset, uint64_t matrix_bytes, uint32_t ggml_type,
        uint32_t ncols, uint32_t nrows, uint32_t row_start, uint32_t row_count, const float *input, uint32_t input_count,
        const int8_t *grid, uint32_t grid_count, float *output, uint32_t output_count, double *io_ms, double *gpu_ms) {
    g_quant_error[0] = '\0';
    if (!model_path || !model_path[0] || !input || !output) { QUANT_ERR("invalid Red Metal mixed-quant arguments"); return 0; }
    if (ggml_type != T_F32 && !pool_quant_supported(ggml_type)) { QUANT_ERR("unsupported GGML type %u", ggml_type); return 0; }
    if (ggml_type == T_IQ2_XS || ggml_type == T_IQ1_M) {      // these two decode through the caller's codebook, as in the reference
        const uint32_t want = ggml_type == T_IQ2_XS ? 512u * 8u : 2048u * 8u;
        if (!grid || grid_count != want) { QUANT_ERR("mixed-quant grid size mismatch: got %u expected %u", grid_count, want); return 0; }
    }
    // a one-shot call binds nothing: it holds the codebook lock from its upload to the end of its kernel instead
    std::unique_lock<std::mutex> grid_lock(caller_grid_mutex(), std::defer_lock);
    if (ggml_type == T_IQ2_XS || ggml_type == T_IQ1_M) {
        grid_lock.lock();
        const hipError_t ge = set_caller_grids_locked(ggml_type == T_IQ2_XS ? grid : nullptr, ggml_type == T_IQ1_M ? grid : nullptr);
        if (ge != hipSuccess) { QUANT_ERR("%s", ge == hipErrorContextAlreadyInUse ? kCodebookConflict : "failed to upload the codebook"); return 0; }
    }
    if (!ncols || ncols % 256u || !nrows || !row_count || row_start >= nrows || row_count > nrows - row_start ||
        input_count != ncols || output_count < row_count) {
        QUANT_ERR("invalid mixed-quant dimensions cols=%u rows=%u start=%u count=%u", ncols, nrows, row_start, row_count);
        return 0;
    }
    const uint64_t rb = pool_row_bytes(ggml_type, ncols);
    if (!rb || (uint64_t)nrows > UINT64_MAX / rb || matrix_bytes != (uint64_t)nrows * rb) {
        QUANT_ERR("matrix byte size mismatch: got %llu expected %llu", (unsigned long long)matrix_bytes, (unsigned long long)((uint64_t)nrows * rb));
        return 0;
    }
    const int fd = open(model_path, O_RDONLY);
    if (fd < 0) { QUANT_ERR("open(%s) failed: %s", model_path, strerror(errno)); return 0; }
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size <= 0) { QUANT_ERR("failed to stat model file: %s", strerror(errno)); close(fd); return 0; }
    std::vector<uint8_t> host((size_t)matrix_bytes);
    const double t_io = now_ms();
    const bool ok = pread_range(fd, (uint64_t)st.st_size, matrix_file_offset, matrix_bytes, host.data(), nullptr, nullptr, g_quant_error, sizeof(g_quant_error));
    const double io = now_ms() - t_io;
    close(fd);
    if (!ok) return 0;
    DevBuf buf;
    const size_t w_bytes = ((size_t)matrix_bytes + 255u) & ~(size_t)255u;
    if (!buf.reserve(w_bytes + ((size_t)ncols + row_count) * sizeof(float))) { QUANT_ERR("failed to allocate mixed quant device buffers"); return 0; }
    uint8_t *dw = static_cast<uint8_t *>(buf.p);
    float *dx = reinterpret_cast<float *>(dw + w_bytes), *dout = dx + ncols;
    hipError_t e = hipMemcpy(dw, host.data(), (size_t)matrix_bytes, hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(dx, input, (size_t)ncols * sizeof(float), hipMemcpyHostToDevice);
    if (e != hipSuccess) { QUANT_ERR("mixed quant upload failed: %s", hipGetErrorString(e)); return 0; }
    const double t_gpu = now_ms();
    e = launch_gemv_rows(ggml_type, dw, ncols, row_start, row_count, dx, dout, nullptr);
    if (e == hipSuccess) e = hipStreamSynchronize(nullptr);
    const double gpu = now_ms() - t_gpu;
    if (e != hipSuccess) { QUANT_ERR("mixed quant HIP command failed: %s", hipGetErrorString(e)); return 0; }
    e = hipMemcpy(output, dout, (size_t)row_count * sizeof(float), hipMemcpyDeviceToHost);
    if (e != hipSuccess) { QUANT_ERR("mixed quant download failed: %s", hipGetErrorString(e)); return 0; }
    if (io_ms) *io_ms = io;
    if (gpu_ms) *gpu_ms = gpu;
    return 1;
}

// ------------------------------------------------------------------ router

int rl_native_router_gpu_f32(const char *model_path, const rl_router_tensor_info *router, const float *input,
        uint32_t input_count, float *logits, uint32_t logits_count, rl_native_router_telemetry *telemetry,
        char *error, size_t error_cap) {
    if (!model_path || !router || !input || !logits || (router->ggml_type != T_F32 && router->ggml_type != T_Q6_K) ||
        router->n_dims != 2u || router->shape[0] > UINT32_MAX || router->shape[1] > UINT32_MAX) {
        set_err(error, error_cap, "invalid HIP router arguments");
        return 0;
    }
    const uint32_t hidden = (uint32_t)router->shape[0], experts = (uint32_t)router->shape[1];
    const uint64_t rb = row_bytes(router->ggml_type, hidden);
    const uint64_t weight_bytes = rb * experts;
    if (!hidden || !experts || !rb || hidden % 256u || input_count != hidden || logits_count < experts ||
        router->tensor_span_bytes < weight_bytes) {
        set_err(error, error_cap, "HIP router shape/span mismatch");
        return 0;
    }
    const int fd = open(model_path, O_RDONLY);
    if (fd < 0) { set_err(error, error_cap, "open GGUF for HIP router failed"); return 0; }
    struct stat st;
    if (fstat(fd, &st) != 0) { close(fd); set_err(error, error_cap, "stat GGUF for HIP router failed"); return 0; }
    std::vector<uint8_t> host((size_t)weight_bytes);
    const double r0 = now_ms();
    char msg[256];
    const bool ok = pread_range(fd, (uint64_t)st.st_size, router->tensor_offset, weight_bytes, host.data(), nullptr, nullptr, msg, sizeof(msg));
    const double r1 = now_ms();
    close(fd);
    if (!ok) { set_err(error, error_cap, "pread router weights failed"); return 0; }
    DevBuf buf;
    const size_t w_bytes = ((size_t)weight_bytes + 255u) & ~(size_t)255u;
    if (!buf.reserve(w_bytes + ((size_t)hidden + experts) * sizeof(float))) { set_err(error, error_cap, "failed to allocate HIP router buffers"); return 0; }
    uint8_t *dw = static_cast<uint8_t *>(buf.p);
    float *dx = reinterpret_cast<float *>(dw + w_bytes), *dl = dx + hidden;
    hipError_t e = hipMemcpy(dw, host.data(), (size_t)weight_bytes, hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(dx, input, (size_t)hidden * sizeof(float), hipMemcpyHostToDevice);
    const double g0 = now_ms();
    if (e == hipSuccess) e = launch_gemv_rows(router->ggml_type, dw, hidden, 0u, experts, dx, dl, nullptr);
    if (e == hipSuccess) e = hipStreamSynchronize(nullptr);
    const double g1 = now_ms();
    if (e == hipSuccess) e = hipMemcpy(logits, dl, (size_t)experts * sizeof(float), hipMemcpyDeviceToHost);
    if (e != hipSuccess) { set_err(error, error_cap, "HIP router command failed: %s", hipGetErrorString(e)); return 0; }
    if (telemetry) { telemetry->read_ms = r1 - r0; telemetry->compute_ms = g1 - g0; }
    if (error && error_cap) error[0] = '\0';
    return 1;
}

int rl_native_router_select_softmax_topk(const float *logits, uint32_t expert_count, uint32_t top_k,
        uint32_t *expert_ids, float *router_weights, float *probabilities, char *error, size_t error_cap) {
    if (!logits || !expert_ids || !router_weights || !expert_count || !top_k || top_k > expert_count) {
        set_err(error, error_cap, "invalid router top-k selection arguments");
        return 0;
    }
    if (expert_count > 1024u || top_k > 16u) { set_err(error, error_cap, "router selection supports at most 1024 experts and top-16"); return 0; }
    DevBuf buf;
    const size_t n_f = (size_t)expert_count * 2u + 1u + 2u * top_k;          // the selection kernel reads one extra logit (the shared gate's)
    if (!buf.reserve(n_f * sizeof(float))) { set_err(error, error_cap, "out of memory for router probabilities"); return 0; }
    float *dl = static_cast<float *>(buf.p), *dp = dl + expert_count + 1u, *dwt = dp + expert_count;
    uint32_t *dids = reinterpret_cast<uint32_t *>(dwt + top_k);
    hipError_t e = hipMemset(dl + expert_count, 0, sizeof(float));
    if (e == hipSuccess) e = hipMemcpy(dl, logits, (size_t)expert_count * sizeof(float), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = launch_select(dl, 1u, expert_count, top_k, dids, dwt, nullptr, dp, nullptr);
    if (e == hipSuccess) e = hipMemcpy(router_weights, dwt, (size_t)top_k * sizeof(float), hipMemcpyDeviceToHost);
    if (e == hipSuccess) e = hipMemcpy(expert_ids, dids, (size_t)top_k * sizeof(uint32_t), hipMemcpyDeviceToHost);
    if (e == hipSuccess && probabilities) e = hipMemcpy(probabilities, dp, (size_t)expert_count * sizeof(float), hipMemcpyDeviceToHost);
    if (e != hipSuccess) { set_err(error, error_cap, "router selection HIP command failed: %s", hipGetErrorString(e)); return 0; }
    for (uint32_t k = 0; k < top_k; ++k)
        if (router_weights[k] != router_weights[k]) {       // NaN marks a softmax whose denominator or selected sum is not finite
            set_err(error, error_cap, "invalid router softmax denominator");
            return 0;
        }
    if (error && error_cap) error[0] = '\0';
    return 1;
}

}  // extern "C"
